"""Python faces of the HIP kernels.

Every function checks on the host that shapes, dtypes and devices are what the kernel and its
grid assume, then launches on torch's current stream.  Tensors are only memory here: no torch
arithmetic runs on the product path except the library matrix product in :func:`linear`.
"""
from __future__ import annotations

import collections

from typing import Optional, Tuple

import torch

from . import lib as _lib
from . import profile as _profile

_DT = {torch.float32: 0, torch.bfloat16: 1}

WINDOW_NONE, WINDOW_CHUNK, WINDOW_SLIDING = 0, 1, 2
ACT_SILU, ACT_GELU_TANH = 1, 2      # the gated unit's activation, as the kernels code it
ACTIVATIONS = {"silu": ACT_SILU, "gelu_tanh": ACT_GELU_TANH}


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"dtype {dtype} is not taken by the kernels (float32 or bfloat16)") from None


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*ts) -> None:
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernel operands must live on the GPU")
            _need(t.is_contiguous(), "kernel operands must be contiguous")


def _i32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None:
        _need(t.dtype == torch.int32, f"{name} must be int32")


def _run(name: str, *args) -> None:
    if _profile._active is not None and _profile._active.depth == 0:
        with _profile.section(name[len("sharpi_"):]):       # a launch outside any section: a class of its own
            return _run(name, *args)
    rc = getattr(_lib.load(), name)(*args)
    if rc != 0:
        what = {1001: "a size or option the kernel does not take", 1002: "launch failed"}.get(rc, f"HIP error {rc}")
        raise KernelError(f"{name}: {what}")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as float32 (the residual stream)."""
    _dev(ids, table, out)
    _i32(ids, "ids")
    _need(ids.dim() == 1 and table.dim() == 2, "embed_gather: ids [T], table [V, H]")
    T, H = ids.shape[0], table.shape[1]
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    _need(out.shape == (T, H) and out.dtype == torch.float32, "embed_gather: out must be float32 [T, H]")
    _run("sharpi_embed_gather", _ptr(ids), _ptr(table), _code(table.dtype), _ptr(out), T, H, float(scale), _stream())
    return out


def scale_softcap(logits: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """logits (float32, contiguous) in place: x * scale, then cap * tanh(x / cap) if cap > 0."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous() and cap >= 0, "scale_softcap: float32 contiguous logits, cap >= 0")
    _run("sharpi_scale_softcap", _ptr(logits), logits.numel(), float(scale), float(cap), _stream())
    return logits


class ExpertSum:
    """A branch output that is still a sum to be formed: row t = sum_j w[t, j] * y[inv_pos[t*k + j]]
    (+ shared[t]); ``weights`` None means ones (scores already applied to the experts' inputs).
    ``add_rmsnorm`` forms it on the fly; ``tensor()`` forms it with a kernel of its own.  Either
    way the sum is rounded once to y's storage type."""

    __slots__ = ("y", "inv_pos", "shared", "n_tokens", "k", "weights")

    def __init__(self, y: torch.Tensor, inv_pos: torch.Tensor, shared: Optional[torch.Tensor], n_tokens: int, k: int,
                 weights: Optional[torch.Tensor] = None):
        _need(y.dim() == 2 and inv_pos.numel() == n_tokens * k, "ExpertSum: y [rows, H], inv_pos [T*k]")
        if shared is not None:
            _need(shared.shape == (n_tokens, y.shape[1]) and shared.dtype == y.dtype and shared.is_contiguous(),
                  "ExpertSum: shared must be contiguous [T, H] of y's dtype")
        if weights is not None:
            _need(weights.numel() == n_tokens * k and weights.dtype == torch.float32 and weights.is_contiguous(),
                  "ExpertSum: weights must be contiguous float32 [T, k]")
        self.y, self.inv_pos, self.shared, self.n_tokens, self.k, self.weights = y, inv_pos, shared, n_tokens, k, weights

    @property
    def shape(self):
        return (self.n_tokens, self.y.shape[1])

    @property
    def dtype(self):
        return self.y.dtype

    def tensor(self) -> torch.Tensor:
        return moe_combine(self.y[: self.n_tokens * self.k], self.inv_pos, self.shared, self.n_tokens, self.k,
                           self.weights)


def add_rmsnorm(h: torch.Tensor, delta, weight: Optional[torch.Tensor], eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, write_back: bool = True,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(h + delta) -> RMSNorm -> out; the sum goes back into h unless rows are gathered.
    delta: a tensor, an ExpertSum, or None."""
    lazy = delta if isinstance(delta, ExpertSum) else None
    if lazy is not None and h.shape[1] % 8 != 0:
        delta, lazy = lazy.tensor(), None          # the kernel folds a sum in only at widths that are multiples of 8
    base = lazy.y if lazy is not None else delta
    _dev(h, base, weight, rows, out, lazy.weights if lazy is not None else None)
    _i32(rows, "rows")
    _need(h.dim() == 2 and h.dtype == torch.float32, "add_rmsnorm: h must be float32 [T, H]")
    T, H = h.shape
    if delta is not None:
        _need(tuple(delta.shape) == tuple(h.shape), f"add_rmsnorm: delta {tuple(delta.shape)} vs h {tuple(h.shape)}")
    if weight is not None:
        _need(weight.shape == (H,), f"add_rmsnorm: weight {tuple(weight.shape)} vs width {H}")
    n_out = T if rows is None else rows.shape[0]
    if rows is not None:
        write_back = False
    if out is None:
        out = torch.empty(n_out, H, dtype=out_dtype, device=h.device)
    _need(out.shape == (n_out, H) and out.dtype == out_dtype, "add_rmsnorm: out has the wrong shape or dtype")
    _run("sharpi_add_rmsnorm", _ptr(h), _ptr(base), _code(base.dtype) if base is not None else 0,
         _ptr(weight), _code(weight.dtype) if weight is not None else 0, _ptr(out), _code(out_dtype), _ptr(rows),
         n_out, H, float(eps), 1 if write_back else 0,
         _ptr(lazy.inv_pos) if lazy is not None else None, _ptr(lazy.shared) if lazy is not None else None,
         _ptr(lazy.weights) if lazy is not None else None, lazy.k if lazy is not None else 0, _stream())
    return out


def gated_act(gate_up: torch.Tensor, scale: Optional[torch.Tensor] = None, act: int = ACT_SILU) -> torch.Tensor:
    """[M, 2I] (gate columns, then up columns) -> act(s*g) * (s*u) [M, I]; act: ACT_SILU or
    ACT_GELU_TANH."""
    _dev(gate_up, scale)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gated_act: input must be [M, 2I]")
    M, I2 = gate_up.shape
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.shape == (M,), "gated_act: scale must be float32 [M]")
    out = torch.empty(M, I2 // 2, dtype=gate_up.dtype, device=gate_up.device)
    _run("sharpi_silu_mul", _ptr(gate_up), _ptr(scale), _ptr(out), _code(gate_up.dtype), M, I2 // 2, int(act), _stream())
    return out


def silu_mul(gate_up: torch.Tensor, scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[M, 2I] (gate columns, then up columns) -> silu(s*g) * (s*u) [M, I]."""
    return gated_act(gate_up, scale, ACT_SILU)


def moe_combine(y: torch.Tensor, inv_pos: torch.Tensor, shared: Optional[torch.Tensor], n_tokens: int,
                k: int, weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_j w[t, j] * y[inv_pos[t*k+j]] (+ shared[t]); weights None: ones."""
    _dev(y, inv_pos, shared, weights)
    _i32(inv_pos, "inv_pos")
    _need(y.dim() == 2 and y.shape[0] == n_tokens * k and inv_pos.numel() == n_tokens * k,
          "moe_combine: y must be [T*k, H] and inv_pos [T*k]")
    H = y.shape[1]
    if shared is not None:
        _need(shared.shape == (n_tokens, H) and shared.dtype == y.dtype, "moe_combine: shared must be [T, H]")
    if weights is not None:
        _need(weights.numel() == n_tokens * k and weights.dtype == torch.float32, "moe_combine: weights must be float32 [T, k]")
    out = torch.empty(n_tokens, H, dtype=y.dtype, device=y.device)
    _run("sharpi_moe_combine", _ptr(y), _ptr(inv_pos), _ptr(shared), _ptr(weights), _ptr(out), _code(y.dtype), n_tokens,
         H, k, _stream())
    return out


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, N] += bias [N] (float32), in place: the sum in float, rounded to x's storage."""
    _dev(x, bias)
    _need(x.dim() == 2 and x.is_contiguous() and bias.dtype == torch.float32 and bias.shape == (x.shape[1],)
          and bias.is_contiguous(), "add_bias: x [T, N] contiguous and bias float32 [N] wanted")
    _run("sharpi_add_bias", _ptr(x), _code(x.dtype), _ptr(bias), x.shape[0], x.shape[1], _stream())
    return x


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _dev(x)
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _run("sharpi_cast", _ptr(x), _code(x.dtype), _ptr(out), _code(dtype), x.numel(), _stream())
    return out


def random_fill(out: torch.Tensor, key: int, kind: int, std: float = 0.02, lo: float = 0.9, hi: float = 1.1) -> torch.Tensor:
    """Fill `out` (float32, bfloat16, or int32 for integers) with the seeded values of
    weights/random_fill.py: element i is a function of (key, i) alone, the same bits as the host makes."""
    from ..weights import random_fill as rf

    _dev(out)
    if kind == rf.FILL_INT:
        _need(out.dtype == torch.int32, "random_fill: integers go into int32")
        code = 0
    else:
        code = _code(out.dtype)
    lo_f, span_f = rf.uniform_fixed(lo, hi)
    _run("sharpi_random_fill", _ptr(out), code, out.numel(), int(key) & ((1 << 64) - 1), int(kind),
         rf.normal_scale(std), lo_f, span_f, _stream())
    return out


# ---------------------------------------------------------------------------
def _cache_shapes_ok(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, hd: int, vd: Optional[int] = None) -> bool:
    """K [pages, nkv, page_size, hd] and V [pages, nkv, vd, page_size] (vd: the values' width, hd unless given)."""
    return (k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == nkv and k_cache.shape[3] == hd
            and v_cache.shape == (k_cache.shape[0], nkv, vd or hd, k_cache.shape[2]))


PAIRS_INTERLEAVED, PAIRS_HALF_SPLIT = 0, 1


def rope_kv(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
            positions: torch.Tensor, inv_freq: Optional[torch.Tensor], qk_norm: bool, eps: float,
            temperature: Optional[Tuple[float, float]], nh: int, nkv: int, hd: int,
            pair_layout: int = PAIRS_INTERLEAVED, bias: Optional[torch.Tensor] = None, vd: Optional[int] = None) -> torch.Tensor:
    """Rotate / norm / scale the heads of qkv [T, (nh+nkv)*hd + nkv*vd] (vd, the values' width, is hd
    unless given); K and V go into the layer's
    cache [pages, nkv, page_size, hd] at slot_mapping; returns q [T, nh*hd].  inv_freq [r/2]
    rotates the first r <= hd elements of every head, in pairs (2i, 2i+1) or (i, i + r/2)
    (``pair_layout``); the rest of the head passes through.  ``bias`` (float32, one value per
    column of qkv) is added to every row first, in float."""
    _dev(qkv, k_cache, v_cache, slot_mapping, positions, inv_freq, bias)
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (qkv.shape[1],) and bias.is_contiguous(),
              "rope_kv: bias must be float32, one value per column of qkv")
    _i32(slot_mapping, "slot_mapping")
    _i32(positions, "positions")
    T = qkv.shape[0]
    vd = int(vd or hd)
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + nkv) * hd + nkv * vd, "rope_kv: qkv must be [T, (nh+nkv)*hd + nkv*vd]")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd, vd), "rope_kv: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, vd, page_size]")
    _need(k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "rope_kv: cache dtype differs from qkv's")
    _need(slot_mapping.shape == (T,) and positions.shape == (T,), "rope_kv: slot_mapping / positions must be [T]")
    rotary_dim = 0
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 1 <= inv_freq.shape[0] <= hd // 2,
              "rope_kv: inv_freq must be float32 [rotary_dim / 2], rotary_dim <= hd")
        rotary_dim = 2 * inv_freq.shape[0]
    _need(pair_layout in (PAIRS_INTERLEAVED, PAIRS_HALF_SPLIT), "rope_kv: pair_layout must be interleaved (0) or half-split (1)")
    page_size = k_cache.shape[2]
    q_out = torch.empty(T, nh * hd, dtype=qkv.dtype, device=qkv.device)
    fs, asc = temperature if temperature is not None else (1.0, 0.0)
    _run("sharpi_rope_kv", _ptr(qkv), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _code(qkv.dtype),
         _ptr(slot_mapping), _ptr(positions), _ptr(inv_freq), _ptr(bias), 1 if qk_norm else 0, float(eps),
         1 if temperature is not None else 0, float(fs), float(asc), T, nh, nkv, hd, vd, page_size, int(pair_layout),
         rotary_dim, _stream())
    return q_out


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      entry_of_token: torch.Tensor, positions: torch.Tensor, window_kind: int, window: int,
                      scale: float, nh: int, nkv: int, hd: int, vd: Optional[int] = None) -> torch.Tensor:
    """Attention of every token of the batch over its request's pages; float arithmetic.  Values
    (and so the output, [T, nh*vd]) may have another width than keys."""
    _dev(q, k_cache, v_cache, block_table, entry_of_token, positions)
    _i32(block_table, "block_table")
    _i32(entry_of_token, "entry_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    vd = int(vd or hd)
    _need(q.shape == (T, nh * hd), "attention: q must be [T, nh*hd]")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd, vd) and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "attention: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, vd, page_size] of q's dtype")
    _need(block_table.dim() == 2, "attention: block_table must be [entries, max_blocks]")
    _need(entry_of_token.shape == (T,) and positions.shape == (T,), "attention: per-token arrays must be [T]")
    out = torch.empty(T, nh * vd, dtype=q.dtype, device=q.device)
    _run("sharpi_attention_generic", _ptr(q), _ptr(k_cache), _ptr(v_cache), _code(q.dtype), _ptr(block_table),
         _ptr(entry_of_token), _ptr(positions), _ptr(out), int(window_kind), int(window), float(scale), T, nh, nkv,
         hd, vd, k_cache.shape[2], block_table.shape[1], k_cache.shape[0], _stream())
    return out


DECODE_RUN_KEYS = _lib.DECODE_RUN_KEYS   # keys per block of the decode kernel (fixed: sums must not depend on the batch)


def decode_max_splits(max_context: int) -> int:
    """Runs of DECODE_RUN_KEYS keys that cover every token of a context of `max_context` tokens,
    whatever its window: runs are aligned to absolute positions, so a token at position p whose
    first visible key is s takes ((p >> 4) - (s >> 4)) // 16 + 1 of them, most for s = 0."""
    return ((max(1, int(max_context)) - 1) >> 4) // (DECODE_RUN_KEYS // 16) + 1


def decode_attention_ok(dtype: torch.dtype, hd: int) -> bool:
    return dtype == torch.bfloat16 and _lib.attention_takes("decode", hd)


def attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                     entry_of_token: torch.Tensor, positions: torch.Tensor, token_list: Optional[torch.Tensor],
                     max_context: int, window_kind: int, window: int, scale: float, nh: int, nkv: int, hd: int,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Split-K flash-decode for the listed tokens (all tokens if token_list is None), each a
    single query over its request's pages.  `max_context` bounds position + 1 of every token."""
    _dev(q, k_cache, v_cache, block_table, entry_of_token, positions, token_list, out)
    _i32(block_table, "block_table")
    _i32(entry_of_token, "entry_of_token")
    _i32(positions, "positions")
    _i32(token_list, "token_list")
    T = q.shape[0]
    _need(q.shape == (T, nh * hd) and decode_attention_ok(q.dtype, hd), "attention_decode: q must be bfloat16 [T, nh*hd], hd a head size the kernel is compiled for")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd) and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "attention_decode: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, hd, page_size] bfloat16")
    _need(block_table.dim() == 2 and entry_of_token.shape == (T,) and positions.shape == (T,),
          "attention_decode: block_table [entries, max_blocks], per-token arrays [T]")
    n_list = T if token_list is None else token_list.shape[0]
    if out is None:
        out = torch.empty_like(q)
    _need(out.shape == q.shape and out.dtype == q.dtype, "attention_decode: out must match q")
    max_splits = decode_max_splits(max_context)
    part_o = torch.empty(n_list * nh * max_splits * hd, dtype=torch.float32, device=q.device)
    part_ml = torch.empty(n_list * nh * max_splits * 2, dtype=torch.float32, device=q.device)
    _run("sharpi_attention_decode", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(entry_of_token),
         _ptr(positions), _ptr(token_list), _ptr(part_o), _ptr(part_ml), _ptr(out), int(window_kind), int(window),
         float(scale), n_list, nh, nkv, hd, k_cache.shape[2], block_table.shape[1], k_cache.shape[0], max_splits,
         _stream())
    return out


PREFILL_TILE_TOKENS = _lib.PREFILL_TILE_TOKENS   # tokens per block of the prefill kernel (32 per wave)


def prefill_attention_ok(dtype: torch.dtype, hd: int) -> bool:
    return dtype == torch.bfloat16 and _lib.attention_takes("prefill", hd)


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      positions: torch.Tensor, tiles: torch.Tensor, window_kind: int, window: int, scale: float,
                      nh: int, nkv: int, hd: int, out: Optional[torch.Tensor] = None,
                      tile_tokens: int = PREFILL_TILE_TOKENS) -> torch.Tensor:
    """Flash attention for the listed tiles: tiles int32 [n, 3] = (entry, first token, rows <=
    tile_tokens), the tokens of a tile consecutive in one entry.  tile_tokens (128, or 64: blocks of
    half the rows, for short prompts) is what the caller cut the tiles to; a row's result does not
    depend on it."""
    _dev(q, k_cache, v_cache, block_table, positions, tiles, out)
    _i32(block_table, "block_table")
    _i32(positions, "positions")
    _i32(tiles, "tiles")
    T = q.shape[0]
    _need(q.shape == (T, nh * hd) and prefill_attention_ok(q.dtype, hd),
          "attention_prefill: q must be bfloat16 [T, nh*hd], hd a head size the kernel is compiled for")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd) and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "attention_prefill: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, hd, page_size] bfloat16")
    _need(block_table.dim() == 2 and positions.shape == (T,) and tiles.dim() == 2 and tiles.shape[1] == 3,
          "attention_prefill: block_table [entries, max_blocks], positions [T], tiles [n, 3]")
    if out is None:
        out = torch.empty_like(q)
    _need(out.shape == q.shape and out.dtype == q.dtype, "attention_prefill: out must match q")
    _run("sharpi_attention_prefill", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(positions),
         _ptr(tiles), _ptr(out), tiles.shape[0], int(tile_tokens), int(window_kind), int(window), float(scale), nh,
         nkv, hd, k_cache.shape[2], block_table.shape[1], k_cache.shape[0], _stream())
    return out


# ---------------------------------------------------------------------------
def gemm_tiled(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [M, K] @ w [N, K]^T with float FMA chains (batch-invariant)."""
    _dev(x, w)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], f"gemm: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    _need(x.dtype == w.dtype, "gemm: x and w must share a dtype")
    out_dtype = out_dtype or x.dtype
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_tiled", _ptr(x), _ptr(w), _ptr(out), _code(x.dtype), _code(out_dtype), M, N, K, None, None, 0,
         _stream())
    return out


# ---------------------------------------------------------------------------
# weights stored for streaming
# ---------------------------------------------------------------------------
class PackedWeight:
    """A bfloat16 matrix [N, K] (or a stack [E, N, K]) stored tile by tile for the decode kernels:
    [N/16][K/128][16 runs of 8 k][16 rows][8], the 4 KB of a (16-row tile, 128-wide unit) in the
    order a wave's lanes read them, so that a wave's load is one contiguous kilobyte.  ``packed``
    has the logical shape but that element order; ``rows`` is the ordinary row-major matrix, kept
    where the library's product (which wants rows) also multiplies by it, else None."""

    __slots__ = ("packed", "rows", "shape", "dtype")

    def __init__(self, packed: torch.Tensor, rows: Optional[torch.Tensor]):
        self.packed, self.rows = packed, rows
        self.shape, self.dtype = packed.shape, packed.dtype

    def dim(self) -> int:
        return len(self.shape)

    def select(self, e: int) -> "PackedWeight":
        """Matrix e of a stack (a view)."""
        return PackedWeight(self.packed[e], self.rows[e] if self.rows is not None else None)


def can_pack(w: torch.Tensor) -> bool:
    return w.dtype == torch.bfloat16 and w.dim() in (2, 3) and w.shape[-2] % 16 == 0 and w.shape[-1] % 128 == 0


def pack_into(dst: torch.Tensor, w: torch.Tensor) -> None:
    """Write w [.., N, K] into dst (same shape, contiguous) in packed order."""
    _need(dst.shape == w.shape and dst.is_contiguous() and can_pack(w), "pack_into: shapes must match and be packable")
    N, K = w.shape[-2], w.shape[-1]
    lead = w.shape[:-2]
    src = w.reshape(*lead, N // 16, 16, K // 128, 16, 8)
    n = len(lead)
    dst.view(*lead, N // 16, K // 128, 16, 16, 8).copy_(src.permute(*range(n), n, n + 2, n + 3, n + 1, n + 4))


_KEEP_ROWS = True


def keep_row_major_copies(keep: bool) -> None:
    """Whether matrices that are packed for the decode kernels also keep their row-major copy for
    the library's product at prompt size (faster prefill, about a tenth more weight memory), or
    only the packed copy (every product then runs in this library's kernels).  Read when weights
    are loaded."""
    global _KEEP_ROWS
    _KEEP_ROWS = bool(keep)


def pack_weight(w: torch.Tensor, keep_rows: Optional[bool] = None):
    """w as a PackedWeight if its shape and type allow it, else w itself."""
    if keep_rows is None:
        keep_rows = _KEEP_ROWS
    if not can_pack(w):
        return w
    packed = torch.empty_like(w, memory_format=torch.contiguous_format)
    pack_into(packed, w)
    return PackedWeight(packed, w if keep_rows else None)


def unpack_weight(w: "PackedWeight") -> torch.Tensor:
    """The row-major matrix of a PackedWeight (a copy unless it is kept)."""
    if w.rows is not None:
        return w.rows
    N, K = w.shape[-2], w.shape[-1]
    lead = tuple(w.shape[:-2])
    n = len(lead)
    src = w.packed.view(*lead, N // 16, K // 128, 16, 16, 8)
    return src.permute(*range(n), n, n + 3, n + 1, n + 2, n + 4).reshape(*lead, N, K).contiguous()


def _unwrap(w):
    """(tensor in the kernel's order, packed?) of a weight given as a tensor or a PackedWeight."""
    return (w.packed, True) if isinstance(w, PackedWeight) else (w, False)


# ---------------------------------------------------------------------------
# the weight-streaming product for few rows (decode)
# ---------------------------------------------------------------------------
SKINNY_MAX_ROWS = 64          # rows the kernel multiplies against one stream of a weight tile (4 blocks of 16)
SKINNY_MAX_ROWS_PLAIN = 32    # plain form: beyond two row blocks the library's product is faster (measured at the
SKINNY_MAX_ROWS_TALL = 32     # model's projection shapes: 18 against 23 us at 32 rows, 28 against 23.5 at 64)
SKINNY_TALL = 65536


def skinny_ok(M: int, N: int, K: int, grouped: bool = False) -> bool:
    limit = SKINNY_MAX_ROWS if grouped else SKINNY_MAX_ROWS_TALL if N >= SKINNY_TALL else SKINNY_MAX_ROWS_PLAIN
    return 0 < M <= limit and K % 128 == 0 and N % 4 == 0


def skinny_plan(N: int, K: int, row_blocks: int = 1, groups: int = 1, act: bool = False):
    """(R, NW): 16-row weight tiles per block and waves per block splitting K (measured on
    MI355X over the projection shapes of the model).  NW, which decides the order of a row's
    sums, depends on nothing (so a row's result does not change with the batch); R only says how
    many independent columns a block computes: two tiles where a block holds one block of 16
    rows (the kernel then keeps two K units in flight per wave), four for wide matrices with
    more rows; one where two would make between one and two blocks per compute unit (some
    units would then stream twice what the others do: 30.7 against 33.3 us for the merged down
    projection of one token)."""
    if row_blocks > 1:
        return (4 if N >= 12288 else 2), 8
    blocks = groups * ((N + 31) // 32)
    units = compute_units()
    return (1 if not act and units < blocks < 2 * units else 2), 8


_COMPUTE_UNITS: dict = {}


def compute_units(device=None) -> int:
    """Compute units of the GPU the launches are laid out for: asked of the device once (the
    MI355X this library is tuned on has 256; so does a host without a GPU, for the tests of the
    launch shapes).  The shape thresholds of ``skinny_plan`` are measured on that part."""
    if not torch.cuda.is_available():
        return 256
    idx = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    if idx not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[idx] = int(torch.cuda.get_device_properties(idx).multi_processor_count)
    return _COMPUTE_UNITS[idx]


def _row_blocks(group_rows: Optional[int]) -> int:
    """16-row blocks of one expert that a grouped launch multiplies at a time: enough for the
    largest group (its bound is the caller's), 1, 2 or 4; larger groups are walked in turns."""
    if not group_rows or group_rows <= 16:
        return 1
    return 2 if group_rows <= 32 else 4


def gemm_skinny(x: torch.Tensor, w, out_dtype: torch.dtype, a_rows: Optional[torch.Tensor] = None,
                offsets: Optional[torch.Tensor] = None, n_rows: Optional[int] = None, R: Optional[int] = None,
                NW: Optional[int] = None, group_rows: Optional[int] = None) -> torch.Tensor:
    """x [M, K] @ w[N, K]^T for M <= 64, or per expert with w [E, N, K] over an expert-sorted row
    list (``group_rows``: a bound on the rows of one expert, if known), on the matrix cores;
    w a tensor (row-major) or a PackedWeight."""
    w, packed = _unwrap(w)
    _dev(x, w, a_rows, offsets)
    _i32(a_rows, "a_rows")
    _i32(offsets, "offsets")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 operands only")
    grouped = offsets is not None
    if grouped:
        _need(w.dim() == 3 and 2 <= offsets.shape[0] <= w.shape[0] + 1,
              "gemm_skinny: grouped needs w [E, N, K] and offsets of at most E + 1 entries")
        E, N, K = offsets.shape[0] - 1, w.shape[1], w.shape[2]
        M = int(n_rows)
        if a_rows is not None:
            _need(a_rows.shape == (M,), "gemm_skinny: a_rows must be [n_rows]")
        else:
            _need(x.shape[0] == M, "gemm_skinny: x must have n_rows rows when not gathered")
    else:
        _need(w.dim() == 2 and a_rows is None, "gemm_skinny: plain needs w [N, K]")
        E, (N, K) = 0, w.shape
        M = x.shape[0]
    _need(x.dim() == 2 and x.shape[1] == K, f"gemm_skinny: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    _need(M > 0 and (grouped or M <= SKINNY_MAX_ROWS) and K % 128 == 0 and N % 4 == 0,
          f"gemm_skinny: shape M={M} N={N} K={K} is not taken (M <= 64 unless grouped, K % 128 == 0, N % 4 == 0)")
    pr, pw = skinny_plan(N, K, _row_blocks(group_rows) if grouped else (M + 15) // 16, max(E, 1))
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_skinny", _ptr(x), _ptr(w), _ptr(out), _code(out_dtype), M, N, K, _ptr(a_rows), _ptr(offsets), E,
         R or pr, NW or pw, 1 if packed else 0, _row_blocks(group_rows) if grouped else 0, _stream())
    return out


def gemm_skinny_swiglu(x: torch.Tensor, w, offsets: torch.Tensor, a_rows: Optional[torch.Tensor],
                       n_rows: int, scale: Optional[torch.Tensor], R: Optional[int] = None,
                       NW: Optional[int] = None, group_rows: Optional[int] = None, act: int = ACT_SILU) -> torch.Tensor:
    """Per expert, silu(s g) * (s u) with (g | u) = x @ w[e]^T rounded to bfloat16, w [E, 2I, K]
    holding gate rows then up rows: the product and the activation in one kernel, for at most
    64 rows.  Returns [n_rows, I] bfloat16."""
    w, packed = _unwrap(w)
    _dev(x, w, a_rows, offsets, scale)
    _i32(a_rows, "a_rows")
    _i32(offsets, "offsets")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny_swiglu: bfloat16 operands only")
    _need(w.dim() == 3 and 2 <= offsets.shape[0] <= w.shape[0] + 1,
          "gemm_skinny_swiglu: w [E, 2I, K] and offsets of at most E + 1 entries")
    E, N, K = offsets.shape[0] - 1, w.shape[1], w.shape[2]
    M = int(n_rows)
    if a_rows is not None:
        _need(a_rows.shape == (M,), "gemm_skinny_swiglu: a_rows must be [n_rows]")
    else:
        _need(x.shape[0] == M, "gemm_skinny_swiglu: x must have n_rows rows when not gathered")
    _need(x.dim() == 2 and x.shape[1] == K, f"gemm_skinny_swiglu: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    _need(M > 0 and K % 128 == 0 and N % 8 == 0,
          f"gemm_skinny_swiglu: shape M={M} N={N} K={K} is not taken (K % 128 == 0, N % 8 == 0)")
    _need(not packed or N % 32 == 0, "gemm_skinny_swiglu: packed weights need gate and up rows in whole 16-row tiles")
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.shape == (M,), "gemm_skinny_swiglu: scale must be float32 [n_rows]")
    pr, pw = skinny_plan(N, K, _row_blocks(group_rows), E, act=True)
    out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=x.device)
    _run("sharpi_gemm_skinny_swiglu", _ptr(x), _ptr(w), _ptr(out), M, N, K, _ptr(a_rows), _ptr(offsets), E,
         _ptr(scale), R or pr, NW or pw, 1 if packed else 0, _row_blocks(group_rows), int(act), _stream())
    return out


ROUTER_MAX_EXPERTS = _lib.ROUTER_MAX_EXPERTS   # experts the routing kernels hold scores for (csrc/router.hip kMaxExperts)
PICKED_MAX_PAIRS = _lib.PICKED_MAX_PAIRS   # (token, pick) pairs of the picked form: one ballot of a wave (csrc/gemm_skinny_kernel.h kMaxPicked)

_COUNTING: dict = {}    # per device: 0, 1, 2, ... (the places of pairs that are stored in their own order)


def counting(n: int, dev: torch.device) -> torch.Tensor:
    """int32 [n] = 0 .. n-1 on the device, from one tensor per device that is made once (outside
    any graph capture)."""
    c = _COUNTING.get(dev)
    if c is None or c.numel() < n:
        _need(not torch.cuda.is_current_stream_capturing(), "counting: the first call on a device must not be captured")
        c = _COUNTING[dev] = torch.arange(max(n, 4096), dtype=torch.int32, device=dev)
    return c[:n]


def picked_ok(n_tokens: int, k: int, N: int, K: int, act: bool, packed: bool) -> bool:
    return (0 < n_tokens * k <= PICKED_MAX_PAIRS and K % 128 == 0
            and N % ((32 if packed else 8) if act else (16 if packed else 4)) == 0)


def gemm_skinny_picked(x: torch.Tensor, w, ids: torch.Tensor, wts: Optional[torch.Tensor], shared: bool, gather: bool,
                       act, out_dtype: torch.dtype) -> torch.Tensor:
    """Per-expert products of a few decode tokens straight from the router's picks ids [T, k]:
    row i of the result is pair i = (token i // k, pick i % k), followed (shared) by one row per
    token through expert E of w [E + 1, N, K].  gather: x [T, K] is read by token, otherwise x is in
    the result's row order.  act (True: SiLU; or an activation's code; False: none): w holds gate
    rows then up rows and the result is act(s g) * (s u) [rows, N/2] with s the pair's weight (wts;
    1 for the shared rows)."""
    act = ACT_SILU if act is True else int(act or 0)
    w, packed = _unwrap(w)
    _dev(x, w, ids, wts)
    _i32(ids, "ids")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny_picked: bfloat16 operands only")
    _need(ids.dim() == 2 and ids.is_contiguous(), "gemm_skinny_picked: ids [T, k]")
    T, k = ids.shape
    E = w.shape[0] - (1 if shared else 0)
    _need(w.dim() == 3 and E >= 1, "gemm_skinny_picked: w [E (+ 1), N, K]")
    N, K = w.shape[1], w.shape[2]
    _need(picked_ok(T, k, N, K, act, packed), f"gemm_skinny_picked: T={T} k={k} N={N} K={K} is not taken")
    rows = T * k + (T if shared else 0)
    _need(x.dim() == 2 and x.shape[1] == K and x.shape[0] == (T if gather else rows),
          f"gemm_skinny_picked: x {tuple(x.shape)} has the wrong shape")
    if wts is not None:
        _need(act and wts.dtype == torch.float32 and wts.shape == ids.shape and wts.is_contiguous(),
              "gemm_skinny_picked: weights are float32 [T, k] and belong to the activation form")
    if act:
        _need(out_dtype == torch.bfloat16, "gemm_skinny_picked: the activation form stores bfloat16")
    # (row blocks: the kernel's own rule; groups: what it launches)
    pr, pw = skinny_plan(N, K, 1 if T * k <= 16 else 2 if T * k <= 32 else 4, min(E, T * k) + (1 if shared else 0), bool(act))
    out = torch.empty(rows, N // 2 if act else N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_skinny_picked", _ptr(x), _ptr(w), _ptr(out), _code(out_dtype), N, K, _ptr(ids), _ptr(wts), T * k, k, E,
         1 if shared else 0, 1 if gather else 0, act, pr, pw, 1 if packed else 0, _stream())
    return out


def linear(x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x W^T.  float32 weights: the float FMA kernel (true 32-bit, whatever x was stored
    as).  bfloat16 weights stored tile by tile (a PackedWeight): the weight-streaming kernel for a
    few rows; beyond, the library's matrix product with float accumulation over the row-major
    copy, as the reference calls a library there (reference:
    src/SharpInference.Cuda/CuBlasInterop.cs:55-68; measured, the library is at the matrix cores'
    peak for plain shapes), or, where only the packed copy is kept, this library's own kernels
    (the few-rows kernel up to 64 rows, the grouped kernel with the matrix as its one group
    beyond)."""
    out_dtype = out_dtype or x.dtype
    if isinstance(w, PackedWeight):
        xb = x if x.dtype == torch.bfloat16 else cast(x, torch.bfloat16)
        _need(xb.dim() == 2 and xb.shape[1] == w.shape[1], f"linear: x {tuple(x.shape)} vs w {tuple(w.shape)}")
        M, (N, K) = xb.shape[0], w.shape
        if skinny_ok(M, N, K):
            return gemm_skinny(xb, w, out_dtype)
        if w.rows is None:
            # only the packed copy is kept (the engine was asked to save memory): this library's own kernels
            if M <= SKINNY_MAX_ROWS:
                return gemm_skinny(xb, w, out_dtype)
            if dense_grouped_ok(M, N, K):
                return linear_many_rows(xb, w, out_dtype)
        w = unpack_weight(w)
    if w.dtype == torch.float32:
        xf = x if x.dtype == torch.float32 else cast(x, torch.float32)
        y = gemm_tiled(xf, w, torch.float32)
        return y if out_dtype == torch.float32 else cast(y, out_dtype)
    _dev(x, w)
    xb = x if x.dtype == torch.bfloat16 else cast(x, torch.bfloat16)
    _need(xb.shape[1] == w.shape[1], f"linear: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    if skinny_ok(xb.shape[0], w.shape[0], w.shape[1]):
        return gemm_skinny(xb, w, out_dtype)
    if out_dtype == torch.bfloat16:
        return torch.mm(xb, w.t())
    return torch.mm(xb, w.t(), out_dtype=torch.float32)


def grouped_gemm(x: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, a_rows: Optional[torch.Tensor],
                 n_rows: int) -> torch.Tensor:
    """Rows [offsets[e], offsets[e+1]) of the expert-sorted list times w[e]^T.
    x rows are read through a_rows when given; w is [E, N, K]; returns [n_rows, N]."""
    _dev(x, w, offsets, a_rows)
    _i32(offsets, "offsets")
    _i32(a_rows, "a_rows")
    _need(w.dim() == 3 and x.dim() == 2 and x.shape[1] == w.shape[2] and x.dtype == w.dtype,
          f"grouped_gemm: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    N, K = w.shape[1], w.shape[2]
    E = offsets.shape[0] - 1          # the weight may hold more experts than the routing has groups
    _need(1 <= E <= w.shape[0], "grouped_gemm: offsets must have at most E + 1 entries")
    if a_rows is not None:
        _need(a_rows.shape == (n_rows,), "grouped_gemm: a_rows must be [n_rows]")
    else:
        _need(x.shape[0] == n_rows, "grouped_gemm: x must have n_rows rows when not gathered")
    out = torch.empty(n_rows, N, dtype=x.dtype, device=x.device)
    _run("sharpi_gemm_tiled", _ptr(x), _ptr(w), _ptr(out), _code(x.dtype), _code(x.dtype), n_rows, N, K, _ptr(a_rows),
         _ptr(offsets), E, _stream())
    return out


# ---------------------------------------------------------------------------
GATE_SIGMOID, GATE_SOFTMAX = 0, 1


def router_topk(x: torch.Tensor, wr: torch.Tensor, k: int, gate: int = GATE_SIGMOID, renorm: bool = False,
                want_gates: bool = False):
    """Router logits in float, gate, k picks (lowest index wins a tie).
    Returns ids int32 [T, k], weights float32 [T, k] (and the gate values [T, E] if asked)."""
    _dev(x, wr)
    _need(x.dim() == 2 and wr.dim() == 2 and x.shape[1] == wr.shape[1], "router: x [T, H], wr [E, H]")
    T, H = x.shape
    E = wr.shape[0]
    ids = torch.empty(T, k, dtype=torch.int32, device=x.device)
    wts = torch.empty(T, k, dtype=torch.float32, device=x.device)
    gates = torch.empty(T, E, dtype=torch.float32, device=x.device) if want_gates else None
    _run("sharpi_router_topk", _ptr(x), _code(x.dtype), _ptr(wr), _code(wr.dtype), _ptr(ids), _ptr(wts), _ptr(gates),
         T, H, E, k, gate, 1 if renorm else 0, _stream())
    return (ids, wts, gates) if want_gates else (ids, wts)


FUSED_NORM_ROUTER_MAX_HIDDEN = _lib.FUSED_NORM_ROUTER_MAX_HIDDEN   # csrc/router.hip kFusedMaxHidden


def norm_router_ok(h: torch.Tensor, delta, out_dtype: torch.dtype) -> bool:
    """Can add_rmsnorm_router take this step?  (a plain bfloat16 delta or none, a width the
    kernel's LDS row holds)"""
    return (out_dtype == torch.bfloat16 and h.shape[1] % 8 == 0 and h.shape[1] <= FUSED_NORM_ROUTER_MAX_HIDDEN
            and (delta is None or (isinstance(delta, torch.Tensor) and delta.dtype == torch.bfloat16
                                   and delta.is_contiguous() and tuple(delta.shape) == tuple(h.shape))))


def add_rmsnorm_router(h: torch.Tensor, delta: Optional[torch.Tensor], weight: Optional[torch.Tensor], eps: float,
                       wr: torch.Tensor, k: int, gate: int = GATE_SIGMOID, renorm: bool = False):
    """add_rmsnorm (the sum goes back into h) and router_topk on its output in one launch, for a
    few tokens: returns (normalised rows bfloat16 [T, H], ids [T, k], weights [T, k]), the bits
    of the two kernels in a row."""
    _dev(h, delta, weight, wr)
    _need(h.dim() == 2 and h.dtype == torch.float32, "add_rmsnorm_router: h must be float32 [T, H]")
    T, H = h.shape
    _need(norm_router_ok(h, delta, torch.bfloat16), "add_rmsnorm_router: bfloat16 rows of a width the kernel holds only")
    if delta is not None:
        _need(tuple(delta.shape) == (T, H) and delta.is_contiguous(), "add_rmsnorm_router: delta must be [T, H]")
    if weight is not None:
        _need(weight.shape == (H,), f"add_rmsnorm_router: weight {tuple(weight.shape)} vs width {H}")
    _need(wr.dim() == 2 and wr.shape[1] == H, "add_rmsnorm_router: wr [E, H]")
    E = wr.shape[0]
    out = torch.empty(T, H, dtype=torch.bfloat16, device=h.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=h.device)
    wts = torch.empty(T, k, dtype=torch.float32, device=h.device)
    _run("sharpi_add_rmsnorm_router", _ptr(h), _ptr(delta), _ptr(weight), _code(weight.dtype) if weight is not None else 0,
         _ptr(out), T, H, float(eps), _ptr(wr), _code(wr.dtype), _ptr(ids), _ptr(wts), E, k, gate, 1 if renorm else 0,
         _stream())
    return out, ids, wts




class Routing:
    """The expert-sorted view of a step's (token, pick) pairs, all on the device."""

    __slots__ = ("n_tokens", "k", "n_experts", "n_groups", "offsets", "sorted_token", "sorted_w", "inv_pos", "plan")

    @property
    def n_rows(self) -> int:
        """Rows of the sorted list: one per (token, pick), plus one per token for a shared group."""
        return self.n_tokens * self.k + (self.n_tokens if self.n_groups > self.n_experts else 0)


_PLAN_INTS: dict = {}


def _new_routing(T: int, k: int, n_experts: int, shared_group: bool, dev) -> Routing:
    rt = Routing()
    rt.n_tokens, rt.k, rt.n_experts = T, k, n_experts
    rt.n_groups = n_experts + (1 if shared_group else 0)
    rows = T * k + (T if shared_group else 0)
    if rt.n_groups not in _PLAN_INTS:
        _PLAN_INTS[rt.n_groups] = _lib.grouped_plan_ints(rt.n_groups)
    n_plan = _PLAN_INTS[rt.n_groups]
    ints = torch.empty(rt.n_groups + 1 + rows + T * k + n_plan, dtype=torch.int32, device=dev)
    o = 0
    rt.offsets = ints[o:o + rt.n_groups + 1]; o += rt.n_groups + 1
    rt.sorted_token = ints[o:o + rows]; o += rows
    rt.inv_pos = ints[o:o + T * k]; o += T * k
    rt.plan = ints[o:o + n_plan]
    rt.sorted_w = torch.empty(rows, dtype=torch.float32, device=dev)
    return rt


def moe_permute(ids: torch.Tensor, wts: torch.Tensor, n_experts: int, shared_group: bool = False) -> Routing:
    """(token, pick) pairs sorted by expert: offsets [E+1], sorted_token, sorted_w, inv_pos, and
    the plan of the grouped product for many rows, which
    says how the experts' row tiles are dealt to the blocks (csrc/grouped_plan.h).  With
    shared_group one more group follows the experts: every token once with weight 1."""
    _dev(ids, wts)
    _i32(ids, "ids")
    _need(ids.shape == wts.shape and wts.dtype == torch.float32 and ids.dim() == 2, "moe_permute: ids/wts [T, k]")
    T, k = ids.shape
    rt = _new_routing(T, k, n_experts, shared_group, ids.device)
    _run("sharpi_moe_permute", _ptr(ids), _ptr(wts), _ptr(rt.offsets), _ptr(rt.sorted_token), _ptr(rt.sorted_w),
         _ptr(rt.inv_pos), _ptr(rt.plan), rt.plan.numel(), T, k, n_experts,
         1 if shared_group else 0, _stream())
    return rt


def route(x: torch.Tensor, wr: torch.Tensor, k: int, gate: int = GATE_SIGMOID, renorm: bool = False,
          shared_group: bool = False):
    """router_topk then moe_permute: (ids, weights, Routing)."""
    ids, wts = router_topk(x, wr, k, gate, renorm)
    return ids, wts, moe_permute(ids, wts, wr.shape[0], shared_group)


def gemm_grouped(x: torch.Tensor, w, rt: Routing, gather: bool, out_dtype: torch.dtype, max_blocks: int = 0) -> torch.Tensor:
    """Per-group products for many rows on the matrix cores (bfloat16): the experts, and the
    always-on group if the routing has one (group E of w).  gather: x rows are read through the
    routing's token list; otherwise x is already in expert-sorted order.  The product's blocks
    stay on their compute units until the work is done; ``max_blocks`` > 0 bounds their number
    (the units left over are for other work running beside the product).  Products that read
    one routing must not run at the same time (they share its plan's ticket counters)."""
    w, packed = _unwrap(w)
    _dev(x, w)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_grouped: bfloat16 operands only")
    _need(w.dim() == 3 and w.shape[0] >= rt.n_groups and x.dim() == 2 and x.shape[1] == w.shape[2],
          f"gemm_grouped: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    E, N, K = w.shape
    _need(K % 64 == 0 and N % 4 == 0, "gemm_grouped: K % 64 == 0 and N % 4 == 0 wanted")
    _need(x.shape[0] == (rt.n_tokens if gather else rt.n_rows), "gemm_grouped: x has the wrong number of rows")
    out = torch.empty(rt.n_rows, N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_grouped", _ptr(x), x.shape[0], _ptr(w), _ptr(out), _code(out_dtype), rt.n_rows, N, K,
         _ptr(rt.sorted_token) if gather else None, _ptr(rt.offsets), _ptr(rt.plan), rt.n_groups,
         1 if packed else 0, int(max_blocks), _stream())
    return out


def gemm_grouped_swiglu(x: torch.Tensor, w, rt: Routing, scale: Optional[torch.Tensor], gather: bool = True,
                        act: int = ACT_SILU, max_blocks: int = 0) -> torch.Tensor:
    """Per group, act(s g) * (s u) with (g | u) = x @ w[e]^T rounded to bfloat16, for many rows: the
    grouped product with the activation (ACT_SILU, ACT_GELU_TANH) in its epilogue.  gather: x rows are read through the
    routing's token list (the order inside a group is whatever the routing kernel made it);
    otherwise x is already in the groups' order.  w [E (+ 1), 2I, K] holds gate rows then up
    rows.  Returns [n_rows, I] bfloat16."""
    w, packed = _unwrap(w)
    _dev(x, w, scale)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_grouped_swiglu: bfloat16 operands only")
    _need(w.dim() == 3 and w.shape[0] >= rt.n_groups and x.dim() == 2 and x.shape[1] == w.shape[2],
          f"gemm_grouped_swiglu: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    E, N, K = w.shape
    _need(K % 64 == 0 and N % 32 == 0, "gemm_grouped_swiglu: K % 64 == 0 and N % 32 == 0 wanted")
    _need(x.shape[0] == (rt.n_tokens if gather else rt.n_rows), "gemm_grouped_swiglu: x has the wrong number of rows")
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.shape == (rt.n_rows,), "gemm_grouped_swiglu: scale must be float32 [n_rows]")
    out = torch.empty(rt.n_rows, N // 2, dtype=torch.bfloat16, device=x.device)
    _run("sharpi_gemm_grouped_swiglu", _ptr(x), x.shape[0], _ptr(w), _ptr(out), rt.n_rows, N, K,
         _ptr(rt.sorted_token) if gather else None, _ptr(rt.offsets), _ptr(rt.plan), rt.n_groups, _ptr(scale), 1 if packed else 0,
         int(act), int(max_blocks), _stream())
    return out


# ---------------------------------------------------------------------------
# plain products of many rows through the grouped kernel (one group: the whole matrix)
# ---------------------------------------------------------------------------
_DENSE_ROUTING: "collections.OrderedDict" = collections.OrderedDict()
_DENSE_ROUTING_KEPT = 64


def _dense_routing(T: int, dev: torch.device) -> Routing:
    """The routing of T rows that all belong to one group: offsets [0, T] and the plan of the
    grouped product for it, made by the routing kernel when a row count is first met and kept for
    the row counts used last (the least recently used one gives way).  Its token list is not used
    (the routing kernel promises no order inside a group): the products read x row by row
    (gather off)."""
    key = (T, dev)
    rt = _DENSE_ROUTING.get(key)
    if rt is None:
        _need(not torch.cuda.is_current_stream_capturing(), "a dense routing's first use must not be captured")
        while len(_DENSE_ROUTING) >= _DENSE_ROUTING_KEPT:
            _DENSE_ROUTING.popitem(last=False)
        ids = torch.zeros(T, 1, dtype=torch.int32, device=dev)
        rt = _DENSE_ROUTING[key] = moe_permute(ids, torch.ones(T, 1, dtype=torch.float32, device=dev), 1)
    else:
        _DENSE_ROUTING.move_to_end(key)
    return rt


def dense_grouped_ok(M: int, N: int, K: int) -> bool:
    return M > 0 and K % 128 == 0 and N % 16 == 0 and N * K <= 0x7fffffff


def linear_many_rows(x: torch.Tensor, w: PackedWeight, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M, K] @ w^T for many rows against a matrix stored tile by tile, on the matrix cores: the
    grouped product with the whole matrix as its one group (row tiles of up to 128 rows whose
    blocks share the weight stream through an XCD's L2)."""
    rt = _dense_routing(x.shape[0], x.device)
    return gemm_grouped(x, PackedWeight(w.packed.unsqueeze(0), None), rt, False, out_dtype)


def swiglu_many_rows(x: torch.Tensor, w_gate_up: PackedWeight, act: int = ACT_SILU) -> torch.Tensor:
    """silu(g) * u with (g | u) = x @ w_gate_up^T rounded to bfloat16, for many rows, the activation
    in the product's epilogue: [M, I] bfloat16."""
    rt = _dense_routing(x.shape[0], x.device)
    return gemm_grouped_swiglu(x, PackedWeight(w_gate_up.packed.unsqueeze(0), None), rt, None, gather=False, act=act)


# ---------------------------------------------------------------------------
def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    _dev(logits)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "argmax: logits must be float32 [rows, vocab]")
    out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
    _run("sharpi_argmax_rows", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _stream())
    return out


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
                top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
                min_p: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(logits, temperature, uniform, top_k, top_p, min_p)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "sample: logits must be float32 [rows, vocab]")
    R = logits.shape[0]
    for name, t, dt in (("temperature", temperature, torch.float32), ("uniform", uniform, torch.float32),
                        ("top_k", top_k, torch.int32), ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32)):
        if t is not None:
            _need(t.shape == (R,) and t.dtype == dt, f"sample: {name} must be {dt} [rows]")
    probs = torch.empty_like(logits)
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _run("sharpi_sample_rows", _ptr(logits), _ptr(probs), _ptr(temperature), _ptr(uniform), _ptr(top_k), _ptr(top_p),
         _ptr(min_p), _ptr(out), R, logits.shape[1], _stream())
    return out


def edit_logits(logits: torch.Tensor, row_offsets: torch.Tensor, ids: torch.Tensor, counts: torch.Tensor,
                bias: torch.Tensor, rep: torch.Tensor, freq: torch.Tensor, pres: torch.Tensor) -> None:
    _dev(logits, row_offsets, ids, counts, bias, rep, freq, pres)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "edit_logits: logits must be float32 [rows, vocab]")
    R = logits.shape[0]
    _i32(row_offsets, "row_offsets"); _i32(ids, "ids"); _i32(counts, "counts")
    _need(row_offsets.shape == (R + 1,), "edit_logits: row_offsets must be [rows + 1]")
    n = ids.shape[0]
    _need(counts.shape == (n,) and bias.shape == (n,) and bias.dtype == torch.float32, "edit_logits: per-entry arrays")
    for t in (rep, freq, pres):
        _need(t.shape == (R,) and t.dtype == torch.float32, "edit_logits: per-row arrays must be float32 [rows]")
    _run("sharpi_edit_logits", _ptr(logits), _ptr(row_offsets), _ptr(ids), _ptr(counts), _ptr(bias), _ptr(rep),
         _ptr(freq), _ptr(pres), R, logits.shape[1], _stream())


# ---------------------------------------------------------------------------
# dispatchers used by the parts
# ---------------------------------------------------------------------------
def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, group, ctx, window_kind: int,
              window: int, scale: float, nh: int, nkv: int, hd: int, vd: Optional[int] = None) -> torch.Tensor:
    """Attention of the step's tokens over their requests' pages (`group`: the cache group's
    block tables, `ctx`: the step).  Values of another width than keys (vd) go through the float kernel."""
    same = vd is None or vd == hd
    if same and decode_attention_ok(q.dtype, hd) and (prefill_attention_ok(q.dtype, hd) or not ctx.n_prefill_tiles):
        # entries of one token: split-K decode kernel; longer entries: flash kernel, a tile of tokens a block
        out = torch.empty_like(q)
        if ctx.n_prefill_tiles:
            attention_prefill(q, k_cache, v_cache, group.block_table, ctx.positions, ctx.prefill_tiles, window_kind,
                              window, scale, nh, nkv, hd, out=out, tile_tokens=ctx.prefill_tile_tokens)
        if ctx.n_decode:
            attention_decode(q, k_cache, v_cache, group.block_table, ctx.entry_of_token, ctx.positions,
                             ctx.decode_tokens, group.max_context, window_kind, window, scale, nh, nkv, hd, out=out)
        return out
    return attention_generic(q, k_cache, v_cache, group.block_table, ctx.entry_of_token, ctx.positions, window_kind,
                             window, scale, nh, nkv, hd, vd)


def grouped_swiglu(x: torch.Tensor, w_gate_up, rt: Routing, out_dtype: torch.dtype, scaled: bool = True,
                   act: int = ACT_SILU, max_blocks: int = 0) -> torch.Tensor:
    """The experts' gate|up products of the routed tokens and their activation,
    act(s g) * (s u) with s the pick's weight (``scaled``; otherwise s = 1): [n_rows, I] in
    expert-sorted order.  On the matrix cores the activation is the product's epilogue (the
    few-rows kernel or the many-rows one); otherwise the product and the activation are two kernels."""
    N, K = w_gate_up.shape[1], w_gate_up.shape[2]
    scale = rt.sorted_w if scaled else None
    if x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out_dtype == torch.bfloat16 and K % 128 == 0:
        if rt.n_tokens <= SKINNY_MAX_ROWS and N % (32 if isinstance(w_gate_up, PackedWeight) else 8) == 0:
            return gemm_skinny_swiglu(x, w_gate_up, rt.offsets, rt.sorted_token, rt.n_rows, scale,
                                      group_rows=rt.n_tokens, act=act)
        if rt.n_tokens > SKINNY_MAX_ROWS and N % 32 == 0:
            return gemm_grouped_swiglu(x, w_gate_up, rt, scale, act=act, max_blocks=max_blocks)
    return gated_act(grouped_linear(x, w_gate_up, rt, True, out_dtype), scale, act)


def grouped_linear(x: torch.Tensor, w, rt: Routing, gather: bool, out_dtype: torch.dtype, max_blocks: int = 0) -> torch.Tensor:
    """Per-expert products over the routing's expert-sorted row list: w [E, N, K] (a tensor or a
    PackedWeight); x rows are read through the token list (gather) or are already in sorted order.
    Returns [n_rows, N]."""
    if x.dtype != w.dtype:
        x = cast(x, w.dtype)
    N, K = w.shape[1], w.shape[2]
    a_rows = rt.sorted_token if gather else None
    if w.dtype == torch.bfloat16 and K % 128 == 0 and N % 4 == 0:
        if rt.n_tokens <= SKINNY_MAX_ROWS:   # no expert has more rows than there are tokens
            return gemm_skinny(x, w, out_dtype, a_rows=a_rows, offsets=rt.offsets, n_rows=rt.n_rows,
                               group_rows=rt.n_tokens)
        return gemm_grouped(x, w, rt, gather, out_dtype, max_blocks=max_blocks)
    y = grouped_gemm(x, w, rt.offsets, a_rows, rt.n_rows)
    return y if y.dtype == out_dtype else cast(y, out_dtype)


# ---------------------------------------------------------------------------
# what the GPU gives at best (measured beside the published peaks)
# ---------------------------------------------------------------------------
def measured_peaks(device="cuda:0", read_bytes: int = 4 << 30, repeats: int = 5) -> dict:
    """{"hbm_gbs": GB/s of a pure read of `read_bytes`, "bf16_tflops": TFLOP/s of a resident loop of
    matrix-core products}: the best of `repeats` runs of two measuring kernels of this library."""
    dev = torch.device(device)
    buf = torch.empty(read_bytes, dtype=torch.uint8, device=dev)
    buf.fill_(1)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = best_mfma = float("inf")
    blocks, iters = 256 * 8, 4096
    import ctypes

    done = ctypes.c_longlong(0)
    for _ in range(repeats + 1):
        a.record()
        _run("sharpi_peak_read", _ptr(buf), read_bytes, _ptr(sink), ctypes.addressof(done), _stream())
        b.record()
        b.synchronize()
        best_read = min(best_read, a.elapsed_time(b))
        a.record()
        _run("sharpi_peak_mfma", _ptr(sink), blocks, iters, _stream())
        b.record()
        b.synchronize()
        best_mfma = min(best_mfma, a.elapsed_time(b))
    flops = blocks * 4 * iters * 8 * (2.0 * 16 * 16 * 32)
    return {"hbm_gbs": done.value / best_read / 1e6, "bf16_tflops": flops / best_mfma / 1e9}
