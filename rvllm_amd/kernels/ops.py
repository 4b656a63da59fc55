"""Python face of the HIP kernels.

Every function takes torch tensors that live on the GPU, checks their shapes
and types on the host, and launches on torch's current stream, so the calls
can be captured in a HIP graph.  Nothing here computes on the CPU or falls
back to a library: if the kernel library cannot be loaded the call raises.
"""

from __future__ import annotations

import ctypes
import functools
import threading
from typing import Optional

import torch

from . import build as _build
from . import signatures as _signatures

_lib = None
_lock = threading.Lock()

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def library():
    """The loaded kernel library; builds it when no current build exists."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.ensure_built()
                try:
                    cdll = ctypes.CDLL(str(path))
                except OSError as e:  # pragma: no cover
                    raise KernelError(f"cannot load the kernel library {path}: {e}") from e
                # every entry point's argument types, from the sources the library was built from
                _lib = _signatures.Library(cdll, _signatures.read_signatures(_build.CSRC))
    return _lib


def library_path() -> Optional[str]:
    p = _build.find_library()
    return str(p) if p else None


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().rv_last_error().decode())


# torch's current stream as a raw handle.  torch.cuda.current_stream() builds a Python object on the way and costs
# some microseconds, a third of the host's time for a step of several hundred launches; the binding below it does not.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


# The entry points' argument types are declared (``signatures.py``), so a call takes plain numbers: an address as an
# int or None, a float as a float.  Building a ctypes object for each of the twenty-odd arguments of a launch cost
# more than the rest of the call.
def _stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}; kernels take float32 and bfloat16") from None


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel arguments must live on the GPU")
            _need(t.is_contiguous(), "kernel arguments must be contiguous")


def _i32(*tensors: torch.Tensor) -> None:
    for t in tensors:
        _need(t.dtype == torch.int32, f"index tensors must be int32, got {t.dtype}")


_c_int, _c_float, _c_ll = int, float, int


V_GROUP = 16  # slots whose values of one dimension lie side by side (RV_V_GROUP of csrc/kv_layout.h)


def _cache_geometry(k_pages: torch.Tensor, v_pages: torch.Tensor, what: str) -> tuple[int, int, int, int]:
    """(pages, kv heads, page size, head size) of a layer's cache: keys are
    ``[pages, kv_heads, page_size, head_dim]``, values are transposed inside
    groups of 16 slots, ``[pages, kv_heads, page_size / 16, head_dim, 16]``."""
    _need(k_pages.dim() == 4 and v_pages.dim() == 5, f"{what}: key pages must have four dimensions, value pages five")
    num_pages, nkv, page_size, hd = k_pages.shape
    _need(page_size % V_GROUP == 0 and tuple(v_pages.shape) == (num_pages, nkv, page_size // V_GROUP, hd, V_GROUP),
          f"{what}: keys are {tuple(k_pages.shape)}, so values must be "
          f"{(num_pages, nkv, page_size // V_GROUP, hd, V_GROUP)} with pages a multiple of {V_GROUP}, "
          f"got {tuple(v_pages.shape)}")
    return num_pages, nkv, page_size, hd


class SlicedSums:
    """The result of a product whose K range was split over blocks, not yet
    added up: 32-bit partial sums ``[slices, rows, width]``.  The kernels that
    consume a product's result (norm + residual add, q/k norm and rotation,
    gated activation) add the slices themselves, in their order, which saves a
    kernel and a rounding; anything else calls ``as_tensor``."""

    def __init__(self, data: torch.Tensor, dtype: torch.dtype):
        self.data = data  # [slices, rows, width] float32
        self.dtype = dtype  # what the product's result would be stored as
        self.slices, self.rows, self.width = data.shape

    @property
    def shape(self):
        return (self.rows, self.width)

    @property
    def device(self):
        return self.data.device

    def as_tensor(self) -> torch.Tensor:
        out = torch.empty((self.rows, self.width), dtype=self.dtype, device=self.data.device)
        _check(library().rv_reduce_slices(_stream(), _ptr(self.data), _ptr(out), _dt(out), _c_int(self.slices),
                                          _c_int(self.rows), _c_int(self.width)))
        return out


class TiledWeight:
    """A bf16 matrix ``[N, K]`` stored for the few-row product: in tiles of 16 rows x 32 columns, each tile's
    1 KB in the order in which the 64 lanes of a matrix-core product hold it, a row of tiles (all of K)
    contiguous, so that a wave reads its share of the matrix as one contiguous stream.  ``rows`` is the same
    matrix row by row, kept for the products that go to the library (more than 64 rows), or None."""

    def __init__(self, rows: torch.Tensor, keep_rows: bool = True):
        _gpu(rows)
        _need(rows.dim() == 2 and rows.dtype == torch.bfloat16, "TiledWeight: a bf16 matrix expected")
        self.n, self.k = rows.shape
        lib = library()
        lib.rv_tile_weight_elements.restype = ctypes.c_longlong
        self.tiles = torch.empty(lib.rv_tile_weight_elements(_c_int(self.n), _c_int(self.k)), dtype=torch.bfloat16,
                                 device=rows.device)
        _check(lib.rv_tile_weight(_stream(), _ptr(rows), _ptr(self.tiles), _c_int(self.n), _c_int(self.k),
                                  _c_ll(rows.stride(0))))
        self.rows = rows if keep_rows else None

    @property
    def shape(self):
        return (self.n, self.k)

    @property
    def dtype(self):
        return torch.bfloat16

    @property
    def device(self):
        return self.tiles.device


def as_tensor(x) -> torch.Tensor:
    """A plain tensor from a tensor or from unreduced ``SlicedSums``."""
    return x.as_tensor() if isinstance(x, (SlicedSums, BranchSum)) else x


def _branch_args(x, what: str):
    """(pointer, slices, slice stride, rows, width, dtype) of a kernel input
    that is a tensor or ``SlicedSums``."""
    if isinstance(x, SlicedSums):
        return _ptr(x.data), x.slices, x.rows * x.width, x.rows, x.width, x.dtype
    _gpu(x)
    _need(x.dim() == 2, f"{what}: a matrix is expected")
    return _ptr(x), 0, 0, x.shape[0], x.shape[1], x.dtype


# --------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
    _gpu(table, ids, out)
    _i32(ids)
    vocab, hidden = table.shape
    n = ids.numel()
    _need(out.shape == (n, hidden), f"embed_gather: out is {tuple(out.shape)}, expected {(n, hidden)}")
    _check(library().rv_embed_gather(_stream(), _ptr(table), _dt(table), _ptr(ids), _ptr(out), _dt(out), _c_int(n),
                                     _c_int(hidden), _c_int(vocab), _c_float(scale)))
    return out


def embed_positions(table: torch.Tensor, pos_table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
                    scale: float, out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale + pos_table[positions[t]], added in 32-bit."""
    _gpu(table, pos_table, ids, positions, out)
    _i32(ids, positions)
    vocab, hidden = table.shape
    n = out.shape[0]
    _need(pos_table.dim() == 2 and pos_table.shape[1] == hidden and pos_table.dtype == table.dtype,
          "embed_positions: the position table must have the token table's width and type")
    _need(out.shape == (n, hidden) and ids.numel() >= n and positions.numel() >= n,
          f"embed_positions: out is {tuple(out.shape)}, ids and positions must cover its rows")
    _check(library().rv_embed_positions(_stream(), _ptr(table), _ptr(pos_table), _dt(table), _ptr(ids), _ptr(positions),
                                        _ptr(out), _dt(out), _c_int(n), _c_int(hidden), _c_int(vocab),
                                        _c_int(pos_table.shape[0]), _c_float(scale)))
    return out


def scalar_rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype: Optional[torch.dtype] = None,
                   out: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row-wise x * rsqrt(mean(x^2) + eps) * gain with one number as the gain.  ``x`` may be the 32-bit residual
    stream of a bf16 model: the result then has ``out_dtype``.  ``rows`` as in ``rmsnorm``."""
    _gpu(x, gain, out, rows)
    _need(x.dim() == 2, "scalar_rmsnorm: a matrix is expected")
    _need(gain.numel() == 1 and gain.dtype in _DT, "scalar_rmsnorm: the gain is one number")
    width = x.shape[1]
    if rows is not None:
        _i32(rows)
    n_rows = x.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype or x.dtype, device=x.device)
    _need(out.shape == (n_rows, width), "scalar_rmsnorm: bad out")
    _check(library().rv_scalar_rmsnorm(_stream(), _ptr(x), _dt(x), _ptr(rows), _ptr(gain),
                                       _c_int(gain.dtype == torch.float32), _ptr(out), _dt(out), _c_int(n_rows),
                                       _c_int(width), _c_float(eps)))
    return out


def residual_mix(x: torch.Tensor, mixer_branch, ff_branch, mult: float, history: Optional[torch.Tensor] = None,
                 terms: int = 0, depth_weights: Optional[torch.Tensor] = None, seed_history: bool = False,
                 next_gain: Optional[torch.Tensor] = None, next_eps: float = 0.0,
                 next_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """The 32-bit residual stream ``x [rows, width]`` takes a layer's two branches, in place:
    X = x + mult * (mixer_branch + ff_branch); with ``history`` (float32 ``[slots, rows, width]``) X is kept as
    entry ``terms - 1`` and x becomes sum_j depth_weights[j] * history[j] over the first ``terms`` entries
    (``seed_history``: entry 0 is x as it came in); otherwise x becomes X.  With ``next_gain`` also returns
    ``scalar_rmsnorm`` of the new x in ``next_dtype``.  A branch is a tensor of the activations' type, unreduced
    ``SlicedSums``, or (the feed-forward's) None."""
    _gpu(x, history, depth_weights, next_gain)
    _need(x.dtype == torch.float32 and x.dim() == 2, "residual_mix: the residual stream is a 32-bit matrix")
    rows, width = x.shape
    aptr, a_slices, a_stride, a_rows, a_width, a_dtype = _branch_args(mixer_branch, "residual_mix")
    _need((a_rows, a_width) == (rows, width), "residual_mix: the mixer's branch must match the residual stream")
    fptr, f_slices, f_stride = None, 0, 0
    if ff_branch is not None:
        fptr, f_slices, f_stride, f_rows, f_width, f_dtype = _branch_args(ff_branch, "residual_mix")
        _need((f_rows, f_width) == (rows, width) and f_dtype == a_dtype,
              "residual_mix: the feed-forward's branch must match the mixer's")
    stride = 0
    if history is not None:
        _need(history.dtype == torch.float32 and history.dim() == 3 and tuple(history.shape[1:]) == (rows, width)
              and 2 <= terms <= history.shape[0], "residual_mix: the history must be 32-bit [slots >= terms, rows, width]")
        _need(depth_weights is not None and depth_weights.numel() == terms and depth_weights.dtype in _DT,
              f"residual_mix: {terms} depth weights expected")
        stride = history.stride(0)
    nxt = None
    if next_gain is not None:
        _need(next_gain.numel() == 1 and next_gain.dtype in _DT, "residual_mix: the next norm's gain is one number")
        nxt = torch.empty((rows, width), dtype=next_dtype or a_dtype, device=x.device)
        _need(nxt.dtype == a_dtype, "residual_mix: the next norm's output has the branches' type")
    _check(library().rv_residual_mix(
        _stream(), _ptr(x), aptr, _c_int(a_slices), _c_ll(a_stride), fptr, _c_int(f_slices), _c_ll(f_stride),
        _c_float(mult), _ptr(history), _c_ll(stride), _c_int(terms), _c_int(int(seed_history)), _ptr(depth_weights),
        _c_int(depth_weights is not None and depth_weights.dtype == torch.float32), _ptr(next_gain),
        _c_int(next_gain is not None and next_gain.dtype == torch.float32), _ptr(nxt), _c_float(next_eps),
        _DT[a_dtype], _c_int(rows), _c_int(width)))
    return nxt


def latent_norm_write(raw: torch.Tensor, col0: int, rank: int, weight: torch.Tensor, eps: float, offset: float,
                      positions: torch.Tensor, token_req: torch.Tensor, block_table: torch.Tensor,
                      k_pages: torch.Tensor, v_pages: torch.Tensor) -> None:
    """Columns ``col0 .. col0 + rank`` of the rows of ``raw``, RMS-normed with ``weight``, into the one-head cache
    ``k_pages`` / ``v_pages`` at each token's position."""
    _gpu(raw, weight, positions, token_req, block_table, k_pages, v_pages)
    _i32(positions, token_req, block_table)
    n = raw.shape[0]
    num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "latent_norm_write")
    _need(nkv == 1 and hd == rank, f"latent_norm_write: the cache must hold one head of {rank} dimensions")
    _need(raw.dim() == 2 and 0 <= col0 and col0 + rank <= raw.shape[1], "latent_norm_write: columns outside the rows")
    _need(k_pages.dtype == raw.dtype and v_pages.dtype == raw.dtype, "latent_norm_write: cache dtype differs")
    _need(weight.shape == (rank,) and weight.dtype in _DT, f"latent_norm_write: the norm's weight must hold {rank} numbers")
    _need(positions.numel() >= n and token_req.numel() >= n, "latent_norm_write: positions/token_req too short")
    _check(library().rv_latent_norm_write(
        _stream(), _ptr(raw), _c_ll(raw.stride(0)), _c_int(col0), _ptr(weight), _c_int(weight.dtype == torch.float32),
        _c_float(eps), _c_float(offset), _ptr(positions), _ptr(token_req), _ptr(block_table),
        _c_int(block_table.shape[1]), _ptr(k_pages), _ptr(v_pages), _c_int(page_size), _c_int(num_pages), _c_int(rank),
        _c_int(n), _dt(raw)))


def gemm_heads(a: torch.Tensor, a_col0: int, w: torch.Tensor, out: Optional[torch.Tensor] = None,
               gate: Optional[torch.Tensor] = None, gate_col0: int = 0) -> torch.Tensor:
    """One product a head, side by side: ``w`` is ``[heads, N, K]``; head h multiplies columns
    ``a_col0 + h K .. + K`` of the rows of ``a`` and fills columns ``h N .. + N`` of ``out [rows, heads N]``.
    With ``gate`` the result is multiplied by sigmoid of the columns ``gate_col0 + ...`` of the rows of ``gate``,
    laid out like ``out``."""
    _need(a.is_cuda and w.is_cuda and a.dim() == 2 and w.dim() == 3 and w.is_contiguous() and a.stride(1) == 1,
          "gemm_heads: rows of inputs and [heads, N, K] matrices on the GPU expected")
    heads, n, k = w.shape
    m = a.shape[0]
    _need(a_col0 >= 0 and a_col0 + heads * k <= a.shape[1], "gemm_heads: the heads' inputs lie outside the rows")
    _need(a.dtype == w.dtype and a.dtype in _DT, "gemm_heads: inputs and matrices of one type, float32 or bfloat16")
    if out is None:
        out = torch.empty((m, heads * n), dtype=a.dtype, device=a.device)
    _need(out.shape == (m, heads * n) and out.dtype == a.dtype and out.is_contiguous(), "gemm_heads: bad out")
    gptr, ldg = None, 0
    if gate is not None:
        _need(gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and gate.dtype == out.dtype
              and gate.shape[0] == m and 0 <= gate_col0 and gate_col0 + heads * n <= gate.shape[1],
              "gemm_heads: the gate must hold the output's columns in its rows")
        gptr, ldg = gate.data_ptr() + gate_col0 * gate.element_size(), gate.stride(0)
    aptr = a.data_ptr() + a_col0 * a.element_size()
    if a.dtype == torch.bfloat16 and _mfma_groups_take(aptr, a.stride(0), w, k):
        _check(library().rv_gemm_groups_mfma(
            _stream(), aptr, _ptr(w), _ptr(out), None, None, _c_int(heads), _c_int(m), _c_int(n), _c_int(k),
            _c_ll(a.stride(0)), _c_ll(k), _c_ll(out.stride(0)), _c_ll(k), _c_ll(n * k), _c_ll(n), gptr, _c_ll(ldg),
            _c_int(0), _c_float(0.0), _c_float(0.0), _c_int(1 if m <= MFMA_GROUPS_FEW_ROWS else 4), _c_int(0)))
        return out
    _check(library().rv_gemm_groups_plain(
        _stream(), aptr, _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), None, None,
        _c_int(heads), _c_int(m), _c_int(n), _c_int(k), _c_ll(a.stride(0)), _c_ll(k), _c_ll(out.stride(0)), _c_ll(k),
        _c_ll(n * k), _c_ll(n), gptr, _c_ll(ldg)))
    return out


# Up to this many rows a wave of the matrix-core kernel for products by group takes one tile of 16 rows against
# one tile of 16 rows of the matrix, so that a launch has waves enough to draw the memory's rate; beyond, four tiles
# of rows against four of the matrix, so that every value read feeds four products.
MFMA_GROUPS_FEW_ROWS = 256


def _mfma_groups_take(aptr: int, lda: int, w: torch.Tensor, k: int) -> bool:
    """Whether the matrix-core kernel for products by group reads these operands: 16 bytes a lane at a time."""
    return k % 8 == 0 and lda % 8 == 0 and aptr % 16 == 0 and w.data_ptr() % 16 == 0


MOE_TILE_ROWS = 64  # rows of one expert that a block of the grouped products takes
MOE_TILE_ROWS_FEW = 16  # the matrix-core kernel's tiles while a step's rows are few


def moe_plan(dtype: torch.dtype, rows: int, *inner_sizes: int) -> tuple[int, bool]:
    """(rows a tile of the sorted order holds, whether the matrix-core kernel multiplies) for a step of ``rows``
    (token, choice) pairs and products whose summed sizes are ``inner_sizes``: bf16 with sizes that are multiples
    of 8 runs on the matrix cores, in tiles of 16 rows while the rows are few and of 64 beyond; everything else in
    tiles of 64 rows on the 32-bit kernel."""
    mfma = dtype == torch.bfloat16 and all(k % 8 == 0 for k in inner_sizes)
    return (MOE_TILE_ROWS_FEW if mfma and rows <= MFMA_GROUPS_FEW_ROWS else MOE_TILE_ROWS), mfma


def moe_capacity(num_tokens: int, top: int, experts: int, tile: int = MOE_TILE_ROWS) -> int:
    """Sorted rows that hold every routing of ``num_tokens * top`` choices: each expert's rows start a tile."""
    return -(-(num_tokens * top + experts * (tile - 1)) // tile) * tile


def moe_route(token_ids: torch.Tensor, num_tokens: int, table: torch.Tensor, experts: int,
              tile: int = MOE_TILE_ROWS) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sorts the step's (token, choice) pairs by the expert that ``table [vocab, top]`` gives the token's id.
    Returns (slot_of ``[tokens * top]``: the sorted row of each pair; row_token ``[capacity]``: the token of each
    sorted row, -1 for filling rows; tile_group ``[capacity / tile]``: the expert of each tile of rows, or -1)."""
    _gpu(token_ids, table)
    _i32(token_ids, table)
    _need(table.dim() == 2 and token_ids.numel() >= num_tokens, "moe_route: a table [vocab, top] and the step's ids")
    vocab, top = table.shape
    capacity = moe_capacity(num_tokens, top, experts, tile)
    slot_of = torch.empty(num_tokens * top, dtype=torch.int32, device=table.device)
    row_token = torch.empty(capacity, dtype=torch.int32, device=table.device)
    tile_group = torch.empty(capacity // tile, dtype=torch.int32, device=table.device)
    _check(library().rv_moe_route(_stream(), _ptr(token_ids), _c_int(num_tokens), _ptr(table), _c_int(vocab),
                                  _c_int(top), _c_int(experts), _c_int(tile), _c_int(capacity), _ptr(slot_of),
                                  _ptr(row_token), _ptr(tile_group)))
    return slot_of, row_token, tile_group


def gemm_experts(a: torch.Tensor, w: torch.Tensor, tile_group: torch.Tensor, row_index: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, tile: int = MOE_TILE_ROWS, mfma: bool = False,
                 glu=None) -> torch.Tensor:
    """``out[r] = a[row_index[r]] @ w[tile_group[r // tile]]^T`` for the sorted rows of ``moe_route``; ``w`` is
    ``[experts, N, K]``.  Without ``row_index`` the rows of ``a`` are the sorted rows themselves.  Rows of tiles
    without an expert are left as they are.  ``tile`` and ``mfma`` are the step's plan (``moe_plan``).  ``glu`` =
    (limit, alpha), on the matrix cores only: ``w`` holds each expert's gate rows and then its up rows, and the
    result is the clamped gated activation of the two products, ``[rows, N / 2]``; ``glu`` = ``"silu"``: the plain
    silu(gate) * up instead."""
    _gpu(a, w, tile_group, row_index, out)
    _i32(tile_group)
    _need(a.dim() == 2 and w.dim() == 3 and a.dtype == w.dtype and a.dtype in _DT and a.shape[1] == w.shape[2],
          "gemm_experts: rows [*, K] against matrices [experts, N, K] of one type expected")
    _need(tile == MOE_TILE_ROWS or (mfma and tile == MOE_TILE_ROWS_FEW), f"gemm_experts: tiles of {tile} rows")
    m = tile_group.numel() * tile
    if row_index is not None:
        _i32(row_index)
        _need(row_index.numel() == m, "gemm_experts: one source row for every sorted row")
    else:
        _need(a.shape[0] == m, "gemm_experts: the rows must be the sorted rows")
    _, n, k = w.shape
    if glu is not None:
        _need(n % 2 == 0 and mfma, "gemm_experts: the activation is applied by the matrix-core kernel")
        n //= 2
    if out is None:
        out = torch.empty((m, n), dtype=a.dtype, device=a.device)
    _need(out.shape == (m, n) and out.dtype == a.dtype, "gemm_experts: bad out")
    if mfma:
        _need(a.dtype == torch.bfloat16 and _mfma_groups_take(a.data_ptr(), a.stride(0), w, k),
              "gemm_experts: the matrix-core kernel takes bf16 and sizes that are multiples of 8")
        kind = 0 if glu is None else (2 if glu == "silu" else 1)
        limit, alpha = glu if kind == 1 else (0.0, 0.0)
        _check(library().rv_gemm_groups_mfma(
            _stream(), _ptr(a), _ptr(w), _ptr(out), _ptr(row_index), _ptr(tile_group), _c_int(0), _c_int(m), _c_int(n),
            _c_int(k), _c_ll(a.stride(0)), _c_ll(k), _c_ll(n), _c_ll(0), _c_ll(w.shape[1] * k), _c_ll(0), None, _c_ll(0),
            _c_int(kind), _c_float(limit), _c_float(alpha), _c_int(tile // 16), _c_int(0)))
        return out
    _check(library().rv_gemm_groups_plain(
        _stream(), _ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), _ptr(row_index), _ptr(tile_group), _c_int(0),
        _c_int(m), _c_int(n), _c_int(k), _c_ll(a.stride(0)), _c_ll(k), _c_ll(n), _c_ll(0), _c_ll(n * k), _c_ll(0),
        None, _c_ll(0)))
    return out


def moe_combine(y: torch.Tensor, slot_of: torch.Tensor, top: int, weight: float, num_tokens: int, shared=None) -> torch.Tensor:
    """out[t] = weight * sum_k y[slot_of[t * top + k]] (+ shared[t]); ``shared`` is a tensor or unreduced
    ``SlicedSums``."""
    _gpu(y, slot_of)
    _i32(slot_of)
    width = y.shape[1]
    _need(slot_of.numel() == num_tokens * top, "moe_combine: one sorted row for every choice")
    sptr, s_slices, s_stride = None, 0, 0
    if shared is not None:
        sptr, s_slices, s_stride, s_rows, s_width, s_dtype = _branch_args(shared, "moe_combine")
        _need((s_rows, s_width) == (num_tokens, width) and s_dtype == y.dtype,
              "moe_combine: the shared expert's output must match")
    out = torch.empty((num_tokens, width), dtype=y.dtype, device=y.device)
    _check(library().rv_moe_combine(_stream(), _ptr(y), _ptr(slot_of), _c_int(top), _c_float(weight), sptr,
                                    _c_int(s_slices), _c_ll(s_stride), _ptr(out), _dt(out), _c_int(num_tokens),
                                    _c_int(width)))
    return out


def clamped_glu(gate_up, limit: float, alpha: float) -> torch.Tensor:
    """g = min(gate, limit), u = clamp(up, -limit, limit): out = g * sigmoid(alpha g) * (u + 1); gates and ups lie in
    the halves of a row of ``gate_up [rows, 2 I]``, a tensor or unreduced ``SlicedSums``."""
    gptr, slices, stride, rows, two_i, dtype = _branch_args(gate_up, "clamped_glu")
    _need(two_i % 2 == 0, "clamped_glu: rows of gates and ups expected")
    inter = two_i // 2
    out = torch.empty((rows, inter), dtype=dtype, device=gate_up.device)
    _check(library().rv_clamped_glu(_stream(), gptr, _c_int(slices), _c_ll(stride), _ptr(out), _dt(out), _c_int(rows),
                                    _c_int(inter), _c_float(limit), _c_float(alpha)))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float,
            out: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row-wise RMSNorm.  With ``rows`` (int32 indices into the rows of a 2-d
    ``x``, all in range: the caller built them) output row r is the norm of
    x[rows[r]]."""
    width = x.shape[-1]
    if rows is not None:
        _need(x.dim() == 2, "rmsnorm: a row index needs a 2-d input")
        _i32(rows)
        n_rows = rows.numel()
        if out is None:
            out = torch.empty((n_rows, width), dtype=x.dtype, device=x.device)
        _need(out.shape == (n_rows, width) and out.dtype == x.dtype, "rmsnorm: bad out")
    else:
        n_rows = x.numel() // width
        if out is None:
            out = torch.empty_like(x)
        _need(out.shape == x.shape and out.dtype == x.dtype, "rmsnorm: out must match x")
    _gpu(x, weight, out, rows)
    _need(weight.shape == (width,), f"rmsnorm: weight is {tuple(weight.shape)}, expected ({width},)")
    _check(library().rv_rmsnorm(_stream(), _ptr(x), _ptr(rows), _ptr(weight), _c_int(weight.dtype == torch.float32),
                                _ptr(out), _dt(x), _c_int(n_rows), _c_int(width), _c_float(eps), _c_float(offset)))
    return out


def add_rmsnorm(branch, weight: torch.Tensor, eps: float, offset: float, residual: torch.Tensor,
                next_weight: Optional[torch.Tensor] = None, next_eps: float = 0.0, next_offset: float = 0.0,
                next_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """residual += rmsnorm(branch); with ``next_weight`` also returns rmsnorm(residual).
    ``branch`` is a tensor or ``SlicedSums``."""
    bptr, slices, stride, rows, width, bdtype = _branch_args(branch, "add_rmsnorm")
    _gpu(weight, residual, next_weight, next_out)
    _need(residual.shape == (rows, width) and residual.dtype == bdtype, "add_rmsnorm: residual must match branch")
    _need(weight.shape == (width,), "add_rmsnorm: bad weight shape")
    if next_weight is not None:
        _need(next_weight.shape == (width,), "add_rmsnorm: bad next weight shape")
        if next_out is None:
            next_out = torch.empty_like(residual)
        _need(next_out.shape == residual.shape and next_out.dtype == residual.dtype, "add_rmsnorm: bad next_out")
    _check(library().rv_add_rmsnorm(
        _stream(), bptr, _c_int(slices), _c_ll(stride), _ptr(weight), _c_int(weight.dtype == torch.float32),
        _ptr(residual), _ptr(next_weight), _c_int(next_weight is not None and next_weight.dtype == torch.float32),
        _ptr(next_out if next_weight is not None else None), _dt(residual), _c_int(rows), _c_int(width), _c_float(eps),
        _c_float(offset), _c_float(next_eps), _c_float(next_offset)))
    return next_out if next_weight is not None else None


ACTIVATIONS = {"gelu_pytorch_tanh": 0, "gelu_tanh": 0, "silu": 1}


# The widths whose gate and up rows may lie in fours (see ``rows_in_fours``): a thread of ``gated_act`` then takes
# its 16 bytes of outputs from 32 neighbouring bytes.
FOURS_WIDTH_MULTIPLE = 8


def rows_in_fours(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The rows of a gate and an up projection ``[I, H]`` as one matrix ``[2 I, H]`` in fours: gates 2q and
    2q + 1, then ups 2q and 2q + 1.  A product against it leaves each gate two places from its up, so that
    ``gemm_bf16_gate_up`` can apply the activation where it holds the sums, and ``gated_act(..., fours=True)``
    reads both from neighbouring bytes."""
    inter, hidden = gate.shape
    _need(up.shape == gate.shape and inter % 2 == 0, "rows_in_fours: two matrices of one shape with an even number of rows")
    return torch.cat([gate.reshape(inter // 2, 2, hidden), up.reshape(inter // 2, 2, hidden)], dim=1).reshape(
        2 * inter, hidden).contiguous()


def gated_act(gate_up, activation: str, out: Optional[torch.Tensor] = None, fours: bool = False) -> torch.Tensor:
    """out[t, i] = act(gate[t, i]) * up[t, i]; ``gate_up`` is a tensor or ``SlicedSums`` whose rows hold the gates
    and then the ups (gate i at i, up i at I + i) or, with ``fours``, what a product against ``rows_in_fours``
    leaves."""
    gptr, slices, stride, rows, two_i, dtype = _branch_args(gate_up, "gated_act")
    _need(two_i % 2 == 0, "gated_act: width must be even")
    inter = two_i // 2
    if out is None:
        out = torch.empty((rows, inter), dtype=dtype, device=gate_up.device)
    _gpu(out)
    _need(out.shape == (rows, inter) and out.dtype == dtype, "gated_act: bad out")
    _need(activation in ACTIVATIONS, f"gated_act: unknown activation {activation!r}")
    _check(library().rv_gated_act(_stream(), gptr, _c_int(slices), _c_ll(stride), _ptr(out), _dt(out), _c_int(rows),
                                  _c_int(inter), _c_int(ACTIVATIONS[activation]), _c_int(int(fours))))
    return out


def add_bias(x, bias: torch.Tensor) -> torch.Tensor:
    """x + bias, row by row: in place for a tensor; unreduced ``SlicedSums`` are added up and the bias with
    them, into a new tensor of the product's type."""
    _gpu(bias)
    if isinstance(x, SlicedSums):
        out = torch.empty((x.rows, x.width), dtype=x.dtype, device=x.device)
        part, slices = x.data, x.slices
    else:
        _gpu(x)
        _need(x.dim() == 2, "add_bias: a matrix is expected")
        out, part, slices = x, None, 0
    rows, width = out.shape
    _need(bias.shape == (width,) and bias.dtype in _DT, f"add_bias: the bias must hold {width} numbers")
    _check(library().rv_add_bias(_stream(), _ptr(out), _dt(out), _ptr(part), _c_int(slices), _ptr(bias),
                                 _c_int(bias.dtype == torch.float32), _c_int(rows), _c_int(width)))
    return out


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    _gpu(logits)
    _need(logits.dtype == torch.float32, "softcap: logits must be float32")
    _check(library().rv_softcap(_stream(), _ptr(logits), _c_ll(logits.numel()), _c_float(cap)))
    return logits


def gemm_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T with 32-bit multiply-adds."""
    _need(a.is_cuda and w.is_cuda and out.is_cuda, "gemm: arguments must live on the GPU")
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: matrices expected")
    m, k = a.shape
    n, k2 = w.shape
    _need(k == k2, f"gemm: inner sizes differ: {k} vs {k2}")
    _need(out.shape == (m, n), f"gemm: out is {tuple(out.shape)}, expected {(m, n)}")
    _need(a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1, "gemm: rows must be contiguous")
    _check(library().rv_gemm_plain(_stream(), _ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), _c_int(m),
                                   _c_int(n), _c_int(k), _c_ll(a.stride(0) if m > 1 else k),
                                   _c_ll(w.stride(0) if n > 1 else k), _c_ll(out.stride(0) if m > 1 else n)))
    return out


def rope_table(inv_freq: torch.Tensor, positions: torch.Tensor, num_tokens: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(cos, sin) of float(position) * inv_freq[i] for the first ``num_tokens``
    positions: two 32-bit tensors ``[num_tokens, len(inv_freq)]``."""
    _gpu(inv_freq, positions)
    _i32(positions)
    _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and inv_freq.numel() > 0, "rope_table: bad inv_freq")
    _need(positions.numel() >= num_tokens, "rope_table: positions too short")
    half = inv_freq.numel()
    cos = torch.empty((num_tokens, half), dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    _check(library().rv_rope_table(_stream(), _ptr(inv_freq), _ptr(positions), _ptr(cos), _ptr(sin), _c_int(num_tokens),
                                   _c_int(half)))
    return cos, sin


def qk_norm_rope_kv_write(qkv, q_out: torch.Tensor, q_weight: Optional[torch.Tensor],
                          k_weight: Optional[torch.Tensor], eps: float, offset: float,
                          rope: Optional[tuple[torch.Tensor, torch.Tensor]], rotary_dim: int, positions: torch.Tensor,
                          token_req: torch.Tensor, block_table: Optional[torch.Tensor],
                          k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], num_q_heads: int,
                          num_kv_heads: int, head_dim: int, write_kv: bool = True,
                          values_by_page=None) -> torch.Tensor:
    """Query/key norm and rotation; queries to ``q_out``, keys and values into the cache (``write_kv``).
    ``values_by_page`` is the step (its q_start, chunk_start, num_requests, max_portion) when extra blocks of the
    same launch are to write the values a page at a time, which pays for prompt portions; the projection must
    then be whole, not partial sums."""
    qptr, slices, stride, n, qkv_width, qkv_dtype = _branch_args(qkv, "qk_norm_rope")
    rope_cos, rope_sin = rope if rope is not None else (None, None)
    _gpu(q_out, q_weight, k_weight, rope_cos, rope_sin, positions, token_req, block_table, k_pages, v_pages)
    _i32(positions, token_req)
    _need(qkv_width == (num_q_heads + 2 * num_kv_heads) * head_dim, "qk_norm_rope: bad qkv shape")
    _need(q_out.shape == (n, num_q_heads * head_dim) and q_out.dtype == qkv_dtype, "qk_norm_rope: bad q_out")
    _need(positions.numel() >= n and token_req.numel() >= n, "qk_norm_rope: positions/token_req too short")
    w_f32 = 0
    if q_weight is not None:
        _need(k_weight is not None and q_weight.shape == (head_dim,) and k_weight.shape == (head_dim,),
              "qk_norm_rope: bad norm weights")
        _need(q_weight.dtype == k_weight.dtype, "qk_norm_rope: norm weights must share a dtype")
        w_f32 = int(q_weight.dtype == torch.float32)
    if rope is not None:
        for table in (rope_cos, rope_sin):
            _need(table.dtype == torch.float32 and table.is_contiguous() and table.shape == (n, rotary_dim // 2),
                  f"qk_norm_rope: the table of cosines and sines must be 32-bit [{n}, {rotary_dim // 2}]")
    page_size = num_pages = width = 0
    by_page = bool(write_kv) and values_by_page is not None
    if by_page:
        _need(slices == 0, "qk_norm_rope: values by pages need a projection that is already added up")
        _gpu(values_by_page.q_start, values_by_page.chunk_start)
        _i32(values_by_page.q_start, values_by_page.chunk_start)
    if write_kv:
        _need(k_pages is not None and v_pages is not None and block_table is not None, "qk_norm_rope: no cache given")
        _i32(block_table)
        num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "qk_norm_rope")
        _need((nkv, hd) == (num_kv_heads, head_dim), "qk_norm_rope: cache pages do not fit the heads")
        _need(k_pages.dtype == qkv_dtype and v_pages.dtype == qkv_dtype, "qk_norm_rope: cache dtype differs")
        width = block_table.shape[1]
    _check(library().rv_qk_norm_rope_kv_write(
        _stream(), qptr, _c_int(slices), _c_ll(stride), _ptr(q_out), _ptr(q_weight), _ptr(k_weight), _c_int(w_f32),
        _c_float(eps),
        _c_float(offset), _ptr(rope_cos), _ptr(rope_sin), _c_int(rotary_dim if rope is not None else 0), _ptr(positions),
        _ptr(token_req), _ptr(block_table), _c_int(width), _ptr(k_pages), _ptr(v_pages), _c_int(page_size),
        _c_int(num_pages), _dt(q_out), _c_int(n), _c_int(num_q_heads), _c_int(num_kv_heads), _c_int(head_dim),
        _c_int((2 if by_page else 1) if write_kv else 0),
        _ptr(values_by_page.q_start if by_page else None), _ptr(values_by_page.chunk_start if by_page else None),
        _c_int(values_by_page.num_requests if by_page else 0), _c_int(values_by_page.max_portion if by_page else 0)))
    return q_out


# Portions of at least this many tokens have their values written a page at a time.
VALUES_BY_PAGE_MIN_PORTION = 16


def _check_sinks(sinks: Optional[torch.Tensor], num_q_heads: int) -> None:
    if sinks is not None:
        _gpu(sinks)
        _need(sinks.dtype == torch.float32 and sinks.shape == (num_q_heads,),
              f"attention: the sinks must be {num_q_heads} 32-bit numbers, one a query head")


def paged_attention_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                            positions: torch.Tensor, token_req: torch.Tensor, out: torch.Tensor, num_q_heads: int,
                            scale: float, window: Optional[int], sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``sinks``: one 32-bit number a query head; head h's sum of exponentials then has one more term
    e^(sinks[h]), with no key and no value."""
    _gpu(q, k_pages, v_pages, block_table, positions, token_req, out)
    _check_sinks(sinks, num_q_heads)
    _i32(block_table, positions, token_req)
    n = q.shape[0]
    num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "attention")
    _need(q.shape == (n, num_q_heads * hd), f"attention: q is {tuple(q.shape)}, expected {(n, num_q_heads * hd)}")
    _need(out.shape == q.shape and out.dtype == q.dtype, "attention: out must match q")
    _need(k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, "attention: cache must match q")
    _need(positions.numel() >= n and token_req.numel() >= n, "attention: positions/token_req too short")
    _check(library().rv_paged_attention_generic(
        _stream(), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(positions), _ptr(token_req), _ptr(out), _dt(q), _c_int(n), _c_int(num_q_heads), _c_int(nkv), _c_int(hd),
        _c_int(page_size), _c_int(num_pages), _c_int(window or 0), _c_float(scale), _ptr(sinks)))
    return out


def paged_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor, step,
                    out: torch.Tensor, num_q_heads: int, scale: float, window: Optional[int],
                    sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of the step's tokens over the cache; picks the kernel.

    The 32-bit path always runs the generic kernel.  bf16 runs the
    matrix-core kernel where it covers the head size and grouping, else the
    generic one."""
    if q.dtype == torch.bfloat16 and mfma_attention_covers(k_pages, v_pages, num_q_heads):
        return paged_attention_mfma(q, k_pages, v_pages, block_table, step, out, num_q_heads, scale, window,
                                    sinks=sinks)
    return paged_attention_generic(q, k_pages, v_pages, block_table, step.positions, step.token_req, out,
                                   num_q_heads, scale, window, sinks)


MFMA_ATTENTION_MAX_HEAD_DIM = 256
MFMA_ATTENTION_MAX_GROUP = 16
# What the split plan of the decode kernel knows about the machine (measured on MI355X at head sizes 64, 128 and
# 256; microseconds): how many of the kernel's waves the machine holds at once is the library's answer for the
# head size at hand (what the kernel's registers allow: one wave a SIMD, 1024 in all, at head size 256; two at
# 128; four at 64); a wave that waits for nobody takes about 1 + head size / 100 for a block of 32 keys (3.6 at
# 256, 2.3 at 128); the waves together stream about 6.3 TB/s; launches and the first reads cost about 7, and the
# merge 0.1 more per split.
_ATTN_WAVE_SLOTS_FALLBACK = 1024
_ATTN_BLOCK_US = (1.0, 0.01)  # a + b * head size
_ATTN_BYTES_PER_US = 6.3e6
_ATTN_FIXED_US = 7.0
_ATTN_FIXED_UNSPLIT_US = 7.0
_ATTN_MERGE_US_PER_SPLIT = 0.1


@functools.lru_cache(maxsize=None)
def attention_wave_slots(head_dim: int) -> int:
    """How many waves of the matrix-core decode kernel for this head size the GPU holds at once."""
    entry = getattr(library(), f"rv_attn_mfma_wave_slots_g{(head_dim // 16 - 1) // 4}", None)
    slots = entry(_c_int(head_dim)) if entry is not None else -1
    return slots if slots > 0 else _ATTN_WAVE_SLOTS_FALLBACK


def shared_head_groups(num_q_heads: int, cache_kv_heads: int) -> int:
    """How many groups the query heads form for the matrix-core attention kernels.  Usually one group a key/value
    head.  Where the cache holds a single head that more than 16 query heads share (latent attention), the heads are
    cut into equal groups of at most 16, each of which reads that one head: the largest divisor of the head count
    that a tile holds."""
    if cache_kv_heads != 1 or num_q_heads <= MFMA_ATTENTION_MAX_GROUP:
        return cache_kv_heads
    group = max(g for g in range(1, MFMA_ATTENTION_MAX_GROUP + 1) if num_q_heads % g == 0)
    return num_q_heads // group


def mfma_attention_covers(k_pages: torch.Tensor, v_pages: torch.Tensor, num_q_heads: int) -> bool:
    _, nkv, page_size, hd = k_pages.shape
    if not (hd % 16 == 0 and hd <= MFMA_ATTENTION_MAX_HEAD_DIM and page_size % 16 == 0 and num_q_heads % nkv == 0):
        return False
    return num_q_heads // shared_head_groups(num_q_heads, nkv) <= MFMA_ATTENTION_MAX_GROUP


@functools.lru_cache(maxsize=4096)
def plan_attention_splits(num_requests: int, max_portion: int, max_context: int, nkv: int, group: int,
                          window: Optional[int], head_dim: int = 256,
                          wave_slots: int = _ATTN_WAVE_SLOTS_FALLBACK) -> tuple[int, int, int]:
    """(tiles per request, number of key splits, keys per split) for the
    matrix-core decode kernel.  A tile is 16 / group_pad tokens of one request
    and one key/value head; its keys are split over waves.

    The number of splits is the one a small model of the machine likes best:
    the waves run in rounds of ``wave_slots`` (``attention_wave_slots``: as
    many as the machine holds at once); a round takes what its longest wave
    takes alone or what its bytes take at full streaming rate, whichever is
    longer; a last round that is not full still takes a wave's whole time,
    which is why 1.3 rounds are worse than 1 or 2; every split adds to the
    merge."""
    group_pad = 1
    while group_pad < group:
        group_pad *= 2
    tokens_per_tile = 16 // group_pad
    tiles = -(-max_portion // tokens_per_tile)
    span = max_context
    if window:
        # first key of a tile rounded down to 32, up to the tile's last token
        span = min(span, window - 1 + 31 + tokens_per_tile)
    blocks = -(-span // 32)
    units = num_requests * tiles * nkv
    block_bytes = 32 * head_dim * 2 * 2  # keys and values of a block, bf16
    block_us = _ATTN_BLOCK_US[0] + _ATTN_BLOCK_US[1] * head_dim
    best = None
    for splits in range(1, min(blocks, 512) + 1):
        per = -(-blocks // splits)  # blocks a split
        if per * (splits - 1) >= blocks:
            continue  # the last split would be empty: the same plan as with fewer splits
        waves = units * splits
        full_rounds, rest = divmod(waves, wave_slots)
        alone = per * block_us
        time = full_rounds * max(alone, wave_slots * per * block_bytes / _ATTN_BYTES_PER_US)
        if rest:  # fewer waves draw less than the full rate: about its square root of their share
            rate = _ATTN_BYTES_PER_US * (rest / wave_slots) ** 0.5
            time += max(alone, rest * per * block_bytes / rate)
        time += _ATTN_FIXED_US + _ATTN_MERGE_US_PER_SPLIT * splits if splits > 1 else _ATTN_FIXED_UNSPLIT_US
        if best is None or time < best[0] * (1.0 - 1e-9):
            best = (time, splits, per * 32)
    _, splits, split_len = best
    return tiles, splits, split_len


# The kernel that gives a tile's key splits to the eight waves of one block and merges them there, with no second
# kernel: worth it while a wave walks few blocks of keys (a window, a short context), and possible while the
# tile's columns fit the block's LDS.
_ATTN_IN_BLOCK_WAVES = 8
_ATTN_IN_BLOCK_LDS = 64 * 1024
_ATTN_IN_BLOCK_MAX_KEY_BLOCKS = 6
_ATTN_IN_BLOCK_MIN_TILES = 256


def plan_attention_in_block(max_portion: int, max_context: int, group: int, window: Optional[int],
                            head_dim: int, num_tiles: Optional[int] = None) -> Optional[tuple[int, int]]:
    """(keys per split, columns of a tile kept in LDS) if the decode kernel is
    to merge a tile's splits inside its block, else None.  With ``num_tiles``
    (requests x tiles x key/value heads) the answer is also None while the
    tiles are too few to fill the machine eight waves each: then the keys
    are better split further, over more waves than a block has."""
    if num_tiles is not None and num_tiles < _ATTN_IN_BLOCK_MIN_TILES:
        return None
    group_pad = 1
    while group_pad < group:
        group_pad *= 2
    tokens_per_tile = 16 // group_pad
    cols = min(max_portion, tokens_per_tile) * group
    if _ATTN_IN_BLOCK_WAVES * cols * (head_dim + 2) * 4 > _ATTN_IN_BLOCK_LDS:
        return None
    span = max_context
    if window:
        span = min(span, window - 1 + 31 + tokens_per_tile)
    per = -(-(-(-span // 32)) // _ATTN_IN_BLOCK_WAVES)  # blocks of 32 keys a wave
    if per > _ATTN_IN_BLOCK_MAX_KEY_BLOCKS:
        return None
    return per * 32, cols


# Portions of at least this many tokens go to the kernel whose blocks share key
# tiles through LDS; shorter ones (decoded tokens above all) to the kernel that
# splits a request's keys over many waves.
PREFILL_MIN_PORTION = 16


# The prompt kernel's long tiles in pieces (``plan_prefill_pieces``), as measured on MI355X (microseconds): a
# block walks a block of 64 keys in 0.85 + head size / 400 (1.5 at 256) and has a fixed cost of some nine such
# blocks (its queries and table read, the first keys waited for, its sums written); merging costs a launch and
# the pieces' sums written and read again.  Pieces are taken where they shorten the launch by a tenth at least.
_PREFILL_BLOCK_US = (0.85, 1.0 / 400.0)
_PREFILL_PIECE_FIXED = 9.0
_PREFILL_MERGE_US = 6.0
_PREFILL_BYTES_PER_US = 5.0e6
_PREFILL_PIECES_GAIN = 1.1
_PREFILL_PIECES_MOST = 32
_PREFILL_PIECE_LEAST = 2  # blocks of keys
_PREFILL_CUT_BELOW = 4    # tiles are cut only while they are fewer than a quarter of the blocks the machine holds


@functools.lru_cache(maxsize=None)
def attention_prefill_block_slots(head_dim: int) -> int:
    """How many blocks of the prompt attention kernel for this head size the GPU holds at once."""
    entry = getattr(library(), f"rv_attn_prefill_block_slots_g{(head_dim // 16 - 1) // 4}", None)
    slots = entry(_c_int(head_dim)) if entry is not None else -1
    return slots if slots > 0 else 256


def plan_prefill_pieces(lengths, starts, tokens_per_tile: int, window: Optional[int], portion_min: int,
                        head_dim: int, nkv: int, block_slots: int = 256) -> tuple[int, int]:
    """(blocks of 64 keys a piece at most, pieces a tile at most) for the prompt kernel in this step; (any, 1)
    means a tile a block.  ``lengths`` and ``starts``: the portions' tokens and first positions;
    ``block_slots``: the kernel's blocks that the machine holds at once.

    A tile (``tokens_per_tile`` tokens of a portion) walks the keys its tokens see in blocks of 64.  While the
    blocks all fit the machine at once, a launch lasts as long as its longest block; beyond, as the blocks'
    work spread over the machine and half a longest block for the uneven end.  Cutting the long tiles shortens
    the longest block, adds blocks with their fixed cost and the merge: it pays where few tiles walk many keys
    (a portion of a hundred tokens deep in a long context: 16 blocks for 256 CUs), not where the tiles fill
    the machine already (a prompt of 2 048 tokens in one portion is as many tiles as there are CUs, and cut
    tiles would wait for a second turn).  The cut that makes the launch shortest by this count is taken."""
    import numpy as np

    whole = (1 << 20, 1)
    lengths = np.asarray(lengths, dtype=np.int64)
    starts = np.asarray(starts, dtype=np.int64)
    taken = lengths >= portion_min
    if not taken.any():
        return whole
    lengths, starts = lengths[taken], starts[taken]
    tiles = -(-lengths // tokens_per_tile)
    of = np.repeat(np.arange(len(lengths)), tiles)  # the request of every tile
    first = np.zeros(len(lengths), dtype=np.int64)
    np.cumsum(tiles[:-1], out=first[1:])
    tok0 = (np.arange(int(tiles.sum())) - first[of]) * tokens_per_tile
    ntok = np.minimum(tokens_per_tile, lengths[of] - tok0)
    p_first = starts[of] + tok0
    kmin = np.maximum(0, p_first - window + 1) if window else np.zeros_like(p_first)
    cost = -(-(p_first + ntok - (kmin & ~31)) // 64)
    total, longest = int(cost.sum()), int(cost.max())
    block_us = _PREFILL_BLOCK_US[0] + _PREFILL_BLOCK_US[1] * head_dim
    if len(cost) * nkv * _PREFILL_CUT_BELOW > block_slots:
        return whole  # measured: where the tiles fill a quarter of the machine or more, pieces gain little or lose

    def launch(piece_max):
        pieces = -(-cost // piece_max)
        blocks = int(pieces.sum()) * nkv
        long_one = -(-longest // -(-longest // piece_max)) + _PREFILL_PIECE_FIXED  # the longest tile's pieces are equal
        if blocks <= block_slots:
            time = long_one * block_us
        else:
            time = ((total * nkv + blocks * _PREFILL_PIECE_FIXED) / block_slots + 0.5 * long_one) * block_us
        cut = int(pieces[pieces > 1].sum())
        if cut:
            time += _PREFILL_MERGE_US + cut * nkv * 2 * 64 * head_dim * 4 / _PREFILL_BYTES_PER_US
        return time

    best = (launch(longest), longest, 1)
    for pieces in range(2, _PREFILL_PIECES_MOST + 1):
        piece_max = -(-longest // pieces)
        if piece_max < _PREFILL_PIECE_LEAST:
            break
        time = launch(piece_max)
        if time < best[0]:
            best = (time, piece_max, -(-longest // piece_max))
    if best[2] > 1 and launch(longest) >= _PREFILL_PIECES_GAIN * best[0]:
        return best[1], best[2]
    return whole


def _prefill_pieces(step, window, tokens_per_tile, tiles, portion_min, hd, nkv, device, forced):
    """(piece_max, pieces_max, room for the pieces' sums) for the prompt kernel in this step; made once a step
    for the layers that agree in window and sizes (``step.shared``).  ``forced``: (piece_max, pieces_max)."""
    shared = getattr(step, "shared", None)
    key = ("prefill_pieces", window, tokens_per_tile, tiles, portion_min, hd, nkv, forced)
    if shared is not None and key in shared:
        return shared[key]
    piece_max, pieces_max = 1 << 20, 1
    if forced is not None:
        piece_max, pieces_max = forced
    else:
        starts = getattr(step, "host_q_start", None)
        first = getattr(step, "host_chunk_start", None)
        if starts is not None and first is not None:
            lengths = [int(starts[i + 1] - starts[i]) for i in range(step.num_requests)]
            piece_max, pieces_max = plan_prefill_pieces(lengths, first, tokens_per_tile, window, portion_min, hd, nkv,
                                                        attention_prefill_block_slots(hd))
    part = None
    if pieces_max > 1:
        part = torch.empty(step.num_requests * tiles * nkv * pieces_max * (64 * hd + 128), dtype=torch.float32,
                           device=device)
    result = (int(piece_max), int(pieces_max), part)
    if shared is not None:
        shared[key] = result
    return result


def paged_attention_mfma(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                         step, out: torch.Tensor, num_q_heads: int, scale: float, window: Optional[int],
                         splits: Optional[tuple[int, int]] = None, prefill_kernel: Optional[bool] = None,
                         in_block: Optional[bool] = None,
                         prefill_pieces: Optional[tuple[int, int]] = None,
                         sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 attention on the matrix cores.  ``splits`` = (number, keys per
    split) overrides the plan, ``prefill_kernel`` the choice of kernel,
    ``in_block`` whether a tile's splits are merged inside one block and
    ``prefill_pieces`` = (blocks of 64 keys a piece at most, pieces a tile at
    most) how the prompt kernel cuts its long tiles (tests use them to force
    every path)."""
    _gpu(q, k_pages, v_pages, block_table, out)
    _i32(block_table)
    _check_sinks(sinks, num_q_heads)
    n = q.shape[0]
    num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "attention")
    _need(q.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16,
          "attention (matrix cores): bfloat16 only")
    _need(mfma_attention_covers(k_pages, v_pages, num_q_heads),
          f"attention (matrix cores): head_dim {hd} must be a multiple of 16 up to {MFMA_ATTENTION_MAX_HEAD_DIM}, "
          f"at most {MFMA_ATTENTION_MAX_GROUP} query heads per key/value head, pages a multiple of 16")
    _need(q.shape == (n, num_q_heads * hd) and out.shape == q.shape and out.dtype == q.dtype,
          "attention (matrix cores): bad q or out shape")
    _need(n == step.num_tokens, "attention (matrix cores): q must hold the step's tokens")
    cache_nkv, nkv = nkv, shared_head_groups(num_q_heads, nkv)  # groups of query heads; they may share the cache's head
    group = num_q_heads // nkv
    group_pad = 1
    while group_pad < group:
        group_pad *= 2
    lib = library()
    suffix = f"g{(hd // 16 - 1) // 4}"

    # which requests go to which kernel
    longest = step.max_portion
    if prefill_kernel is None:
        use_prefill = longest >= PREFILL_MIN_PORTION
        portion_min = PREFILL_MIN_PORTION
    else:
        use_prefill, portion_min = prefill_kernel, 1
    shortest_rest = 0  # longest portion left to the split-key kernel
    if use_prefill and portion_min > 1:
        starts = getattr(step, "host_q_start", None)
        if starts is None:
            starts = step.q_start.cpu().numpy()
        lengths = [int(starts[i + 1] - starts[i]) for i in range(step.num_requests)]
        shortest_rest = max([x for x in lengths if x < portion_min], default=0)
    elif not use_prefill:
        shortest_rest = longest

    if use_prefill:
        tokens_per_block = 64 // group_pad
        tiles = -(-longest // tokens_per_block)
        piece_max, pieces_max, part = _prefill_pieces(step, window, tokens_per_block, tiles, portion_min, hd, nkv,
                                                      q.device, prefill_pieces)
        entry = getattr(lib, f"rv_attn_prefill_{suffix}")
        _check(entry(_stream(), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                     _c_int(block_table.shape[1]), _ptr(step.q_start), _ptr(step.chunk_start), _ptr(out), _c_int(n),
                     _c_int(step.num_requests), _c_int(tiles), _c_int(num_q_heads), _c_int(nkv), _c_int(hd),
                     _c_int(page_size), _c_int(num_pages), _c_int(window or 0), _c_int(portion_min), _c_float(scale),
                     _c_int(piece_max), _c_int(pieces_max), _ptr(part), _ptr(sinks), _c_int(cache_nkv)))
    if shortest_rest > 0:
        tiles, num_splits, split_len = plan_attention_splits(step.num_requests, shortest_rest, step.max_context, nkv,
                                                             group, window, hd, attention_wave_slots(hd))
        block_cols = 0
        merged = None
        if in_block is not False:
            merged = plan_attention_in_block(shortest_rest, step.max_context, group, window, hd,
                                             None if in_block else step.num_requests * tiles * nkv)
        if in_block:
            _need(merged is not None, "attention: these keys or columns are too many to merge inside a block")
        if merged is not None and (splits is None or in_block):
            num_splits, (split_len, block_cols) = _ATTN_IN_BLOCK_WAVES, merged
        elif splits is not None:
            num_splits, split_len = splits
            need = -(-step.max_context // 32) * 32
            _need(window is not None or num_splits * split_len >= need,
                  "attention: the splits do not cover the context")
        part_o = part_ml = None
        if num_splits > 1 and block_cols == 0:
            units = step.num_requests * tiles * nkv * num_splits
            part_o = torch.empty(units * 16 * hd, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(units * 32, dtype=torch.float32, device=q.device)
        entry = getattr(lib, f"rv_attn_mfma_{suffix}")
        _check(entry(_stream(), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                     _c_int(block_table.shape[1]), _ptr(step.q_start), _ptr(step.chunk_start), _ptr(step.token_req),
                     _ptr(out), _ptr(part_o), _ptr(part_ml), _c_int(n), _c_int(step.num_requests), _c_int(tiles),
                     _c_int(num_q_heads), _c_int(nkv), _c_int(hd), _c_int(page_size), _c_int(num_pages),
                     _c_int(window or 0), _c_int(num_splits), _c_int(split_len),
                     _c_int(portion_min - 1 if use_prefill else 0), _c_int(block_cols), _c_float(scale), _ptr(sinks),
                     _c_int(cache_nkv)))
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _gpu(logits, out)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: float32 [rows, vocab] expected")
    rows, vocab = logits.shape
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    parts = library().rv_argmax_parts(_c_int(vocab))
    ws_val = torch.empty(rows * parts, dtype=torch.float32, device=logits.device)
    ws_idx = torch.empty(rows * parts, dtype=torch.int32, device=logits.device)
    _check(library().rv_argmax(_stream(), _ptr(logits), _c_int(rows), _c_int(vocab), _c_ll(vocab), _ptr(ws_val),
                               _ptr(ws_idx), _ptr(out)))
    return out


def advance_decode(step, chosen: torch.Tensor) -> None:
    """A step of decoded tokens becomes the next one on the device: request b's
    next token is ``chosen[b]``, one position on.  ``step`` is the step's batch
    (token b belongs to request b); its arrays are changed in place."""
    n = step.num_requests
    _need(step.num_tokens == n and step.max_portion == 1, "advance_decode: a step of single decoded tokens expected")
    _gpu(chosen, step.token_ids, step.positions, step.chunk_start, step.context_len)
    _i32(chosen, step.token_ids, step.positions, step.chunk_start, step.context_len)
    _need(chosen.numel() == n, "advance_decode: one chosen token per request expected")
    _check(library().rv_advance_decode(_stream(), _ptr(chosen), _ptr(step.token_ids), _ptr(step.positions),
                                       _ptr(step.chunk_start), _ptr(step.context_len), _c_int(n)))


def copy_rows_to_device(dst: torch.Tensor, src: torch.Tensor, rows: int, cols: int) -> None:
    """``dst[:rows, :cols] = src[:rows, :cols]`` from a pinned host matrix to a device matrix of the same element
    size as one strided copy in the current stream's order (rows far apart, as a step's block tables are: only
    the pages that the step's requests hold travel)."""
    _gpu(dst)
    _need(not src.is_cuda and src.is_pinned(), "copy_rows: the source must be pinned host memory")
    _need(dst.dim() == 2 and src.dim() == 2 and dst.element_size() == src.element_size()
          and dst.stride(1) == 1 and src.stride(1) == 1, "copy_rows: two matrices with rows of the same elements expected")
    _need(0 <= rows <= min(dst.shape[0], src.shape[0]) and 0 <= cols <= min(dst.shape[1], src.shape[1]),
          f"copy_rows: {rows} x {cols} does not fit {tuple(src.shape)} -> {tuple(dst.shape)}")
    e = dst.element_size()
    _check(library().rv_copy_rows_to_device(_stream(), _ptr(dst), _c_ll(dst.stride(0) * e), _ptr(src),
                                            _c_ll(src.stride(0) * e), _c_ll(cols * e), _c_ll(rows)))


def topk_select(logits: torch.Tensor, k: int, inv_temp: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The k largest logits of every row, times 1/T, with their ids (unordered)."""
    _gpu(logits, inv_temp)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "topk_select: float32 [rows, vocab] expected")
    rows, vocab = logits.shape
    _need(inv_temp.dtype == torch.float32 and inv_temp.numel() == rows, "topk_select: one 1/T per row expected")
    vals = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    idx = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    parts = library().rv_topk_parts(_c_int(vocab))
    cand_val = cand_idx = None
    if parts > 1:  # the parts' candidates, from which the row's are selected
        cand_val = torch.empty((rows, parts * k), dtype=torch.float32, device=logits.device)
        cand_idx = torch.empty((rows, parts * k), dtype=torch.int32, device=logits.device)
    _check(library().rv_topk_select(_stream(), _ptr(logits), _c_int(rows), _c_int(vocab), _c_ll(vocab), _c_int(k),
                                    _ptr(inv_temp), _ptr(vals), _ptr(idx), _ptr(cand_val), _ptr(cand_idx)))
    return vals, idx


def draw(vals: torch.Tensor, ids: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, rng_state: torch.Tensor,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token a row from the candidates ``vals, ids [rows, k]`` of ``topk_select``, drawn on the device as the
    host draws (``sampling.sampler.sample_rows``): ``top_k`` int32 and ``top_p`` float64 a row, ``rng_state`` int64
    a row, each request's SplitMix64 state, which moves one draw on.  -1 for a row one of whose own ``top_k``
    candidates is no finite number.  A row with ``top_k`` -1 draws nothing: it gets the largest candidate that is
    a number, the lower id among equals, as ``argmax`` gives it."""
    _gpu(vals, ids, top_k, top_p, rng_state, out)
    rows, k = vals.shape
    _need(vals.dtype == torch.float32 and ids.dtype == torch.int32 and ids.shape == vals.shape,
          "draw: float32 values and int32 ids [rows, k] expected")
    _need(top_k.dtype == torch.int32 and top_p.dtype == torch.float64 and rng_state.dtype == torch.int64
          and top_k.numel() == rows and top_p.numel() == rows and rng_state.numel() == rows,
          "draw: top_k int32, top_p float64 and rng_state int64, one a row, expected")
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=vals.device)
    _need(out.dtype == torch.int32 and out.numel() == rows, "draw: int32 out, one a row, expected")
    _check(library().rv_draw(_stream(), _ptr(vals), _ptr(ids), _c_int(rows), _c_int(k), _ptr(top_k), _ptr(top_p),
                             _ptr(rng_state), _ptr(out)))
    return out


def gemm_bf16(x: torch.Tensor, w, out: Optional[torch.Tensor] = None,
              out_dtype: Optional[torch.dtype] = None, sliced_ok: bool = False):
    """out = x @ w^T on the matrix cores for bf16 inputs; None when no
    hand-written kernel covers the shape (the caller then uses another path).
    ``w`` is a matrix ``[N, K]`` or a ``TiledWeight``.

    Products with up to 64 rows run the kernel that is built around reading
    ``w`` once.  A 32-bit result of more rows (logits at many positions) runs
    it over blocks of 64 rows; a bf16 result of more rows is left to the
    library product.  With ``sliced_ok`` a product whose K range is split over
    blocks returns its partial sums as ``SlicedSums`` instead of adding them."""
    m, k = x.shape
    tiled = isinstance(w, TiledWeight)
    n = w.shape[0]
    out_dtype = out.dtype if out is not None else (out_dtype or x.dtype)
    if k % 8 or x.stride(1) != 1 or (out is not None and out.stride(1) != 1):
        return None
    if (m > 1 and x.stride(0) % 8) or x.data_ptr() % 16:
        return None
    if not tiled and (w.stride(1) != 1 or (n > 1 and w.stride(0) % 8) or w.data_ptr() % 16):
        return None
    if m > SKINNY_MAX_ROWS and out_dtype != torch.float32:
        return None
    _need(x.is_cuda and w.device.type == "cuda", "gemm: arguments must live on the GPU")
    _need(w.shape[1] == k and (out is None or out.shape == (m, n)), "gemm: shapes do not fit")
    lib = library()
    ldx = x.stride(0) if m > 1 else k
    ldw = 0 if tiled else (w.stride(0) if n > 1 else k)
    wptr = _ptr(w.tiles if tiled else w)
    slices = lib.rv_gemm_skinny_slices(_c_int(n), _c_int(k))
    if sliced_ok and out is None and slices > 1 and m <= SKINNY_MAX_ROWS:
        part = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
        _check(lib.rv_gemm_skinny(_stream(), _ptr(x), wptr, None, _dt(x), _ptr(part), _c_int(m), _c_int(n),
                                  _c_int(k), _c_ll(ldx), _c_ll(ldw), _c_ll(n), _c_int(0), _c_int(int(tiled))))
        return SlicedSums(part, out_dtype)
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    ldc = out.stride(0) if m > 1 else n
    rows_max = min(m, SKINNY_MAX_ROWS)
    part = torch.empty(slices * rows_max * n, dtype=torch.float32, device=x.device) if slices > 1 else None
    for m0 in range(0, m, SKINNY_MAX_ROWS):
        rows = min(SKINNY_MAX_ROWS, m - m0)
        _check(lib.rv_gemm_skinny(_stream(), ctypes.c_void_p(x.data_ptr() + m0 * ldx * 2), wptr,
                                  ctypes.c_void_p(out.data_ptr() + m0 * ldc * out.element_size()), _dt(out),
                                  _ptr(part), _c_int(rows), _c_int(n), _c_int(k), _c_ll(ldx), _c_ll(ldw),
                                  _c_ll(ldc), _c_int(1), _c_int(int(tiled))))
    return out


SKINNY_MAX_ROWS = 64

# ---- products of many rows: the library's --------------------------------------------------------------------
LIBRARY_WORKSPACE_BYTES = 64 << 20
_library_workspaces: dict = {}
_library_tuning = False


def library_workspace(device) -> torch.Tensor:
    """The device memory that the library's algorithms may use, one allocation a device, made at first use."""
    device = torch.device(device)
    index = torch.cuda.current_device() if device.index is None else device.index
    ws = _library_workspaces.get(index)
    if ws is None:
        ws = _library_workspaces[index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def set_library_tuning(on: bool) -> None:
    """While on, ``library_gemm`` first times the library's algorithms for every shape it has not tuned yet and
    keeps the fastest (a second or so a shape, with a wait for the device): for warm-up runs, never inside a
    recording."""
    global _library_tuning
    _library_tuning = bool(on)


def _library_args(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor):
    m, k = x.shape
    n = w.shape[0]
    bf16 = torch.bfloat16
    out_f32 = out.dtype is torch.float32
    if not (x.is_cuda and w.is_cuda and out.is_cuda and x.dtype is bf16 and w.dtype is bf16
            and (out.dtype is bf16 or out_f32)
            and w.dim() == 2 and w.shape[1] == k and out.dim() == 2 and out.shape[0] == m and out.shape[1] == n
            and x.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1):
        _need(x.is_cuda and w.is_cuda and out.is_cuda, "library product: arguments must live on the GPU")
        _need(x.dtype == bf16 and w.dtype == bf16 and out.dtype in (bf16, torch.float32),
              "library product: bfloat16 operands, a bfloat16 or float32 result")
        _need(w.dim() == 2 and out.dim() == 2 and w.shape[1] == k and tuple(out.shape) == (m, n),
              f"library product: shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
        _need(False, "library product: rows must be contiguous")
    ws = _library_workspaces.get(x.device.index)
    if ws is None:
        ws = library_workspace(x.device)
    return (x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k, x.stride(0) if m > 1 else k,
            w.stride(0) if n > 1 else k, out.stride(0) if m > 1 else n, ws.data_ptr(), LIBRARY_WORKSPACE_BYTES), int(out_f32)


# The matrices that products of many rows may meet, by shape: tuning a shape takes them in turn (``rv_lt_tune``), so
# that its timed calls read from memory as a step's calls do.  Weak references: a model that goes takes its own along.
_library_matrices: dict = {}


def library_matrix_register(w: torch.Tensor) -> None:
    """Tells the tuning of the library's products that ``w`` ([N, K], bf16, on the GPU) is one of the matrices of
    its shape: a part calls it for every matrix it keeps row by row."""
    import weakref

    if w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.stride(1) == 1:
        key = (w.device.index, w.shape[0], w.shape[1], w.stride(0))
        known = _library_matrices.setdefault(key, [])
        if len(known) >= 1024:  # models come and go: forget the ones that went
            known[:] = [ref for ref in known if ref() is not None]
        known.append(weakref.ref(w))


def _library_matrices_like(w: torch.Tensor):
    """(a C array of the addresses of the registered matrices of ``w``'s shape that are still there, their number);
    (None, 0) if there is none but ``w`` itself."""
    key = (w.device.index, w.shape[0], w.shape[1], w.stride(0))
    alive = [t for t in (ref() for ref in _library_matrices.get(key, ())) if t is not None]
    _library_matrices[key] = [ref for ref in _library_matrices.get(key, ()) if ref() is not None]
    addresses = sorted({t.data_ptr() for t in alive} | {w.data_ptr()})
    if len(addresses) < 2:
        return None, 0
    return (ctypes.c_void_p * len(addresses))(*addresses), len(addresses)


def library_gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> Optional[torch.Tensor]:
    """out[M, N] = x[M, K] @ w[N, K]^T, x and w in bf16, out in bf16 or (logits) float32, with 32-bit sums, by
    hipBLASLt (``csrc/library_gemm.hip``): the product of more rows than the few-row kernel takes.  A shape keeps its plan; see ``set_library_tuning``.
    None, with nothing done, for a shape that the library has no algorithm for."""
    args, out_f32 = _library_args(x, w, out)
    lib = library()
    if _library_tuning:
        others, count = _library_matrices_like(w)
        _check(min(0, lib.rv_lt_tune(_stream(), *args, _c_int(LIBRARY_TUNE_BUDGET_MS), others, _c_int(count), out_f32)))
    status = lib.rv_lt_gemm(_stream(), *args, out_f32)
    if status == 2:  # the library has no algorithm for this shape: nothing ran
        return None
    _check(status)
    return out


LIBRARY_TUNE_BUDGET_MS = 3000
# The environment variable that names a file of tuned plans: ``ModelRunner.warm_up`` reads it before it tunes and
# writes it afterwards, so that a later start finds its shapes tuned.
LIBRARY_PLANS_ENV = "RVLLM_AMD_LIBRARY_PLANS"


def _library_plans_key(device) -> dict:
    """What a file of plans holds for: an algorithm's index means something only to one version of the library on
    one kind of device."""
    kind = ctypes.create_string_buffer(128)
    with torch.cuda.device(device):
        _check(library().rv_lt_device_kind(kind, _c_int(len(kind))))
        return {"device": kind.value.decode(), "hipblaslt": int(library().rv_lt_version())}


def library_plans_save(path: str, device) -> int:
    """Writes the tuned shapes of ``device`` (shape, strides, the algorithm's index, its time, 1 for a 32-bit result) to ``path`` as JSON,
    over what the file held; the number of shapes written."""
    import json
    import os

    lib = library()
    plans = []
    with torch.cuda.device(device):
        while True:
            m, n, k, index, f32 = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            ldx, ldw, ldc = ctypes.c_longlong(), ctypes.c_longlong(), ctypes.c_longlong()
            us = ctypes.c_float()
            if not lib.rv_lt_tuned_plan(_c_int(len(plans)), ctypes.byref(m), ctypes.byref(n), ctypes.byref(k),
                                        ctypes.byref(ldx), ctypes.byref(ldw), ctypes.byref(ldc), ctypes.byref(index),
                                        ctypes.byref(us), ctypes.byref(f32)):
                break
            plans.append([m.value, n.value, k.value, ldx.value, ldw.value, ldc.value, index.value, round(us.value, 2),
                          f32.value])
        doc = dict(_library_plans_key(device), plans=sorted(plans))
    tmp = f"{path}.{os.getpid()}.tmp"
    with open(tmp, "w") as f:
        json.dump(doc, f, indent=0)
    os.replace(tmp, path)
    return len(plans)


def library_plans_load(path: str, device) -> int:
    """Takes the plans of a file written by ``library_plans_save``: the number of shapes that now count as tuned.
    A file that is missing, unreadable, or of another device or version of the library gives 0 and changes nothing;
    so does a plan that the library does not take."""
    import json

    try:
        with open(path) as f:
            doc = json.load(f)
        plans = [(int(m), int(n), int(k), int(ldx), int(ldw), int(ldc), int(index), float(us), int(f32))
                 for m, n, k, ldx, ldw, ldc, index, us, f32 in doc["plans"]]
    except (OSError, ValueError, KeyError, TypeError):
        return 0
    lib = library()
    taken = 0
    with torch.cuda.device(device):
        if {key: doc.get(key) for key in ("device", "hipblaslt")} != _library_plans_key(device):
            return 0
        room = library_workspace(torch.device(device)).numel()
        for m, n, k, ldx, ldw, ldc, index, us, f32 in plans:
            status = lib.rv_lt_take_plan(_c_int(m), _c_int(n), _c_int(k), _c_ll(ldx), _c_ll(ldw), _c_ll(ldc),
                                         _c_int(index), _c_float(us), _c_ll(room), _c_int(f32))
            if status == 0:
                taken += 1  # anything else: the library does not know the algorithm, or refuses the shape; not taken
    return taken


def library_plan_info(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> tuple[int, int, float]:
    """(1 tuned / 2 a tuned neighbour's algorithm: the nearest row count within one and a half times with the same
    matrix / 0 the library's first suggestion / -1 never seen, the algorithm's index, the time it was tuned to in
    microseconds) for the shape of this product."""
    args, out_f32 = _library_args(x, w, out)
    index, us = ctypes.c_int(-1), ctypes.c_float(0.0)
    state = library().rv_lt_plan_info(*args[3:9], ctypes.byref(index), ctypes.byref(us), out_f32)
    return state, index.value, us.value


def probe_read(data: torch.Tensor, blocks: int = 2048) -> torch.Tensor:
    """Reads ``data`` once with a kernel that does nothing else (a measurement of the memory's read rate);
    returns 64 words folded from what was read."""
    _gpu(data)
    nbytes = data.numel() * data.element_size()
    _need(nbytes % 16 == 0 and data.data_ptr() % 16 == 0, "probe_read: 16-byte aligned data of a multiple of 16 bytes")
    out = torch.zeros(64, dtype=torch.int32, device=data.device)
    _check(library().rv_probe_read(_stream(), _ptr(data), _c_ll(nbytes), _ptr(out), _c_int(blocks)))
    return out


def gemm_bf16_gate_up(x: torch.Tensor, w_fours, activation: str):
    """act(x @ gate^T) * (x @ up^T) in one kernel, for a bf16 ``x`` of at most 64 rows and ``w_fours`` =
    ``rows_in_fours(gate, up)`` (as a matrix or a ``TiledWeight``): the product applies the activation where it
    holds the sums, which saves a kernel and a pass over memory.  None when the kernel does not cover the case
    (rows, alignment, a shape whose product is split along K): the caller then multiplies and applies
    ``gated_act(..., fours=True)``."""
    if x.dtype != torch.bfloat16 or w_fours.dtype != torch.bfloat16:
        return None
    m, k = x.shape
    tiled = isinstance(w_fours, TiledWeight)
    n = w_fours.shape[0]
    if m < 1 or m > SKINNY_MAX_ROWS or w_fours.shape[1] != k or k % 8 or n % 4 or x.stride(1) != 1:
        return None
    if (m > 1 and x.stride(0) % 8) or x.data_ptr() % 16:
        return None
    if not tiled and (w_fours.stride(1) != 1 or (n > 1 and w_fours.stride(0) % 8) or w_fours.data_ptr() % 16):
        return None
    _need(x.is_cuda and w_fours.device.type == "cuda", "gemm: arguments must live on the GPU")
    _need(activation in ACTIVATIONS, f"gemm_bf16_gate_up: unknown activation {activation!r}")
    lib = library()
    if lib.rv_gemm_skinny_slices(_c_int(n), _c_int(k)) != 1:
        return None
    out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    _check(lib.rv_gemm_skinny_gate_up(_stream(), _ptr(x), _ptr(w_fours.tiles if tiled else w_fours), _ptr(out), _dt(out),
                                      _c_int(m), _c_int(n), _c_int(k), _c_ll(x.stride(0) if m > 1 else k),
                                      _c_ll(0 if tiled else (w_fours.stride(0) if n > 1 else k)), _c_ll(n // 2),
                                      _c_int(ACTIVATIONS[activation]), _c_int(int(tiled))))
    return out


# ---- a 32-bit residual stream between sandwiched branches ---------------------------------------------------
def rmsnorm_cast(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float, out_dtype: torch.dtype,
                 out: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row-wise RMSNorm whose result has another type than its input (a 32-bit residual stream, activations in
    bf16).  ``rows`` as in ``rmsnorm``."""
    _gpu(x, weight, out, rows)
    _need(x.dim() == 2, "rmsnorm_cast: a matrix is expected")
    width = x.shape[1]
    _need(weight.shape == (width,) and weight.dtype in _DT, f"rmsnorm_cast: the weight must hold {width} numbers")
    if rows is not None:
        _i32(rows)
    n_rows = x.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=x.device)
    _need(out.shape == (n_rows, width) and out.dtype == out_dtype, "rmsnorm_cast: bad out")
    _check(library().rv_rmsnorm_cast(_stream(), _ptr(x), _dt(x), _ptr(rows), _ptr(weight),
                                     _c_int(weight.dtype == torch.float32), _ptr(out), _dt(out), _c_int(n_rows),
                                     _c_int(width), _c_float(eps), _c_float(offset)))
    return out


class BranchSum:
    """a * x + b * y for two branches of one shape and type (tensors or unreduced ``SlicedSums``), not added up yet:
    the kernel that norms a branch and adds it to the residual stream takes the two as they are
    (``add_rmsnorm_scaled``); anything else calls ``as_tensor``."""

    def __init__(self, x, y, a: float, b: float):
        self.x, self.y, self.a, self.b = x, y, float(a), float(b)
        self.shape, self.device = x.shape, x.device
        self.dtype = x.dtype

    def as_tensor(self) -> torch.Tensor:
        return weighted_sum(self.x, self.y, self.a, self.b).as_tensor()


def add_rmsnorm_scaled(branch, weight: torch.Tensor, eps: float, offset: float, scale: Optional[torch.Tensor],
                       residual: torch.Tensor, next_weight: Optional[torch.Tensor] = None, next_eps: float = 0.0,
                       next_offset: float = 0.0) -> Optional[torch.Tensor]:
    """residual += rmsnorm(branch) * scale on a 32-bit ``residual``; ``scale`` is one number a channel or None.
    With ``next_weight`` also returns rmsnorm(residual) in the branch's type.  ``branch`` is a tensor of the
    activations' type, ``SlicedSums``, or a ``BranchSum`` of two of these."""
    second, wa, wb = None, 1.0, 0.0
    if isinstance(branch, BranchSum):
        branch, second, wa, wb = branch.x, branch.y, branch.a, branch.b
    bptr, slices, stride, rows, width, bdtype = _branch_args(branch, "add_rmsnorm_scaled")
    sptr, s_slices, s_stride = None, 0, 0
    if second is not None:
        sptr, s_slices, s_stride, s_rows, s_width, s_dtype = _branch_args(second, "add_rmsnorm_scaled")
        _need((s_rows, s_width, s_dtype) == (rows, width, bdtype), "add_rmsnorm_scaled: two branches of one shape and type")
    _gpu(weight, scale, residual, next_weight)
    _need(residual.shape == (rows, width) and residual.dtype == torch.float32,
          "add_rmsnorm_scaled: the residual stream is a 32-bit matrix of the branch's shape")
    _need(weight.shape == (width,) and weight.dtype in _DT, "add_rmsnorm_scaled: bad weight")
    _need(scale is None or (scale.shape == (width,) and scale.dtype in _DT), "add_rmsnorm_scaled: bad scale")
    nxt = None
    if next_weight is not None:
        _need(next_weight.shape == (width,) and next_weight.dtype in _DT, "add_rmsnorm_scaled: bad next weight")
        nxt = torch.empty((rows, width), dtype=bdtype, device=residual.device)
    _check(library().rv_add_rmsnorm_scaled(
        _stream(), bptr, _c_int(slices), _c_ll(stride), sptr, _c_int(s_slices), _c_ll(s_stride), _c_float(wa),
        _c_float(wb), _ptr(weight), _c_int(weight.dtype == torch.float32),
        _ptr(scale), _c_int(scale is not None and scale.dtype == torch.float32), _ptr(residual), _ptr(next_weight),
        _c_int(next_weight is not None and next_weight.dtype == torch.float32), _ptr(nxt), _DT[bdtype], _c_int(rows),
        _c_int(width), _c_float(eps), _c_float(offset), _c_float(next_eps), _c_float(next_offset)))
    return nxt


def scale_(x: torch.Tensor, a: float) -> torch.Tensor:
    """x *= a for a 32-bit tensor, in place."""
    _gpu(x)
    _need(x.dtype == torch.float32, "scale_: a 32-bit tensor expected")
    _check(library().rv_scale_f32(_stream(), _ptr(x), _c_ll(x.numel()), _c_float(a)))
    return x


def weighted_sum(x, y, a: float, b: float) -> SlicedSums:
    """a * x + b * y for two branches (tensors of one type or unreduced ``SlicedSums``), added in 32-bit and left
    32-bit: the result is handed on as the one slice of a product's partial sums."""
    xptr, x_slices, x_stride, rows, width, dtype = _branch_args(x, "weighted_sum")
    yptr, y_slices, y_stride, y_rows, y_width, y_dtype = _branch_args(y, "weighted_sum")
    _need((rows, width, dtype) == (y_rows, y_width, y_dtype), "weighted_sum: two branches of one shape and type")
    out = torch.empty((1, rows, width), dtype=torch.float32, device=x.device)
    _check(library().rv_weighted_sum(_stream(), xptr, _c_int(x_slices), _c_ll(x_stride), yptr, _c_int(y_slices),
                                     _c_ll(y_stride), _c_float(a), _c_float(b), _ptr(out), _DT[dtype], _c_int(rows),
                                     _c_int(width)))
    return SlicedSums(out, dtype)


# ---- attention with a partial rotation in halves, a norm after it, values that are the keys ----------------------
NORM_NONE, NORM_BEFORE_ROTATION, NORM_AFTER_ROTATION = 0, 1, 2


def rotate_norm_write(proj: torch.Tensor, q_col: int, k_col: int, v_col: Optional[int], q_out: torch.Tensor,
                      q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float, offset: float,
                      norm_mode: int, rope: Optional[tuple[torch.Tensor, torch.Tensor]], rotary_dim: int,
                      positions: torch.Tensor, token_req: torch.Tensor, block_table: Optional[torch.Tensor],
                      k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], num_q_heads: int,
                      num_kv_heads: int, head_dim: int, write_kv: bool = True,
                      bias: Optional[torch.Tensor] = None, norm_dim: Optional[int] = None) -> torch.Tensor:
    """Queries and keys from the rows of ``proj`` (queries from column ``q_col``, keys from ``k_col``, values from
    ``v_col`` or, with None, the keys as they stand there): rotation of the first ``rotary_dim`` dimensions of a
    head, dimension i paired with i + rotary_dim / 2; per-head RMS norm before or after it (``norm_mode``), with
    the weights or without; queries to ``q_out``, keys and values into the cache.  ``bias``: one 32-bit number
    for every column of ``proj``, added to queries, keys and values as they are read.  ``norm_dim``: the head's own
    size where it is stored wider than it is, with zeros behind (the norm's mean runs over that many)."""
    norm_dim = head_dim if norm_dim is None else int(norm_dim)
    cos, sin = rope if rope is not None else (None, None)
    _gpu(q_out, q_weight, k_weight, cos, sin, positions, token_req, block_table, k_pages, v_pages, bias)
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (proj.shape[1],)),
          "rotate_norm_write: the bias holds a 32-bit number for every column of the rows")
    _need(proj.is_cuda and proj.dim() == 2 and proj.stride(1) == 1, "rotate_norm_write: rows of projections expected")
    _i32(positions, token_req)
    n = proj.shape[0]
    q_size, kv_size = num_q_heads * head_dim, num_kv_heads * head_dim
    cols = proj.shape[1]
    _need(0 <= q_col and q_col + q_size <= cols and 0 <= k_col and k_col + kv_size <= cols
          and (v_col is None or (0 <= v_col and v_col + kv_size <= cols)), "rotate_norm_write: columns outside the rows")
    _need(q_out.shape == (n, q_size) and q_out.dtype == proj.dtype, "rotate_norm_write: bad q_out")
    _need(positions.numel() >= n and token_req.numel() >= n, "rotate_norm_write: positions/token_req too short")
    w_f32 = 0
    if q_weight is not None or k_weight is not None:
        _need(q_weight is not None and k_weight is not None and q_weight.shape == (norm_dim,)
              and k_weight.shape == (norm_dim,) and q_weight.dtype == k_weight.dtype and q_weight.dtype in _DT,
              "rotate_norm_write: bad norm weights")
        w_f32 = int(q_weight.dtype == torch.float32)
    rot = rotary_dim if rope is not None else 0
    if rot:
        for table in (cos, sin):
            _need(table.dtype == torch.float32 and table.shape == (n, rot // 2),
                  f"rotate_norm_write: the table of cosines and sines must be 32-bit [{n}, {rot // 2}]")
    page_size = num_pages = width = 0
    if write_kv:
        _need(k_pages is not None and v_pages is not None and block_table is not None, "rotate_norm_write: no cache given")
        _i32(block_table)
        num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "rotate_norm_write")
        _need((nkv, hd) == (num_kv_heads, head_dim), "rotate_norm_write: cache pages do not fit the heads")
        _need(k_pages.dtype == proj.dtype and v_pages.dtype == proj.dtype, "rotate_norm_write: cache dtype differs")
        width = block_table.shape[1]
    _check(library().rv_rotate_norm_write(
        _stream(), _ptr(proj), _c_ll(proj.stride(0)), _c_int(q_col), _c_int(k_col), _c_int(-1 if v_col is None else v_col),
        _ptr(bias), _ptr(q_out), _ptr(q_weight), _ptr(k_weight), _c_int(w_f32), _c_float(eps), _c_float(offset), _c_int(norm_mode),
        _ptr(cos), _ptr(sin), _c_int(rot), _ptr(positions), _ptr(token_req), _ptr(block_table), _c_int(width),
        _ptr(k_pages), _ptr(v_pages), _c_int(page_size), _c_int(num_pages), _dt(proj), _c_int(n), _c_int(num_q_heads),
        _c_int(num_kv_heads), _c_int(head_dim), _c_int(int(write_kv)), _c_int(norm_dim)))
    return q_out


GATE_ACTS = {"sigmoid": 0, "silu": 1}


def gate_mul_(a: torch.Tensor, gate: torch.Tensor, gate_col0: int, act: str) -> torch.Tensor:
    """a[t, c] *= act(gate[t, gate_col0 + c]), in place; ``act`` is ``sigmoid`` or ``silu``."""
    _gpu(a)
    _need(gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and a.dim() == 2 and gate.dtype == a.dtype
          and gate.shape[0] == a.shape[0] and 0 <= gate_col0 and gate_col0 + a.shape[1] <= gate.shape[1],
          "gate_mul: the gate must hold the columns of a in its rows")
    _need(act in GATE_ACTS, f"gate_mul: unknown activation {act!r}")
    _check(library().rv_gate_mul(_stream(), _ptr(a), gate.data_ptr() + gate_col0 * gate.element_size(),
                                 _c_ll(gate.stride(0)), _dt(a), _c_int(a.shape[0]), _c_int(a.shape[1]),
                                 _c_int(GATE_ACTS[act])))
    return a


# ---- mixers with a state of fixed size ------------------------------------------------------------------------
def _state_args(slots: torch.Tensor, what: str) -> int:
    _gpu(slots)
    _need(slots.dim() == 2 and slots.dtype == torch.float32, f"{what}: the state slots are 32-bit [slots, size]")
    return slots.stride(0)


CONV_ACTS = {"silu": 0, "none": 1}


def causal_conv(x: torch.Tensor, col0: int, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor],
                slots: torch.Tensor, state_off: int, step, out: torch.Tensor, out_col0: int = 0, group: int = 64,
                unit_eps: Optional[float] = None, scaled_groups: int = 0, group_scale: float = 1.0,
                state_ld: Optional[int] = None, move_state: bool = False, act: str = "silu") -> torch.Tensor:
    """Short causal convolution over time and ``act`` (``silu``, or ``none``) for the channels ``col0 .. col0 + channels`` of the rows of
    ``x``: ``weight`` is float32 ``[channels, taps]`` (the last tap is the token's own), ``bias`` float32 or None.
    The inputs before a request's first token of the step come from its state slot (``taps - 1`` rows of
    ``channels`` floats from ``state_off`` on), which this call only reads (``conv_state_update`` moves it on).
    Results go to the columns ``out_col0 ...`` of ``out`` (float32 or the type of ``x``).  With ``unit_eps`` every
    group of ``group`` channels is divided by sqrt(sum of squares + unit_eps), and the first ``scaled_groups``
    groups are multiplied by ``group_scale``.  ``state_ld``: the channels a row of the state holds, when these
    are a part of them (``state_off`` then points at this part's first channel).  ``move_state``: the kernel also
    moves the state on for these channels; only for a step in which every request brings exactly one token (see
    ``conv_moves_state``), where it replaces ``conv_state_update``."""
    _gpu(weight, bias)
    _need(act in CONV_ACTS, f"causal_conv: unknown activation {act!r}")
    _need(not move_state or step.max_portion == 1, "causal_conv: the state moves with the kernel in steps of single tokens only")
    state_ld = channels if state_ld is None else int(state_ld)
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and out.is_cuda and out.dim() == 2 and out.stride(1) == 1,
          "causal_conv: rows expected")
    n = x.shape[0]
    _need(n == step.num_tokens and out.shape[0] == n, "causal_conv: the rows must be the step's tokens")
    _need(0 <= col0 and col0 + channels <= x.shape[1] and 0 <= out_col0 and out_col0 + channels <= out.shape[1],
          "causal_conv: channels outside the rows")
    _need(weight.dim() == 2 and weight.shape[0] == channels and weight.dtype == torch.float32
          and (bias is None or (bias.shape == (channels,) and bias.dtype == torch.float32)),
          "causal_conv: float32 weights [channels, taps] and bias [channels] expected")
    _need(out.dtype == torch.float32 or out.dtype == x.dtype, "causal_conv: the result is float32 or of the input's type")
    taps = weight.shape[1]
    stride = _state_args(slots, "causal_conv")
    _need(state_ld >= channels and 0 <= state_off
          and state_off + max(0, taps - 2) * state_ld + (channels if taps > 1 else 0) <= slots.shape[1],
          "causal_conv: the state lies outside the slot")
    _check(library().rv_causal_conv(
        _stream(), x.data_ptr() + col0 * x.element_size(), _dt(x), _c_ll(x.stride(0)), _ptr(weight), _ptr(bias),
        _c_int(taps), _ptr(slots), _c_ll(stride), _c_ll(state_off), _c_int(state_ld), _ptr(step.positions),
        _ptr(step.token_req), _ptr(step.q_start), _ptr(step.chunk_start), _ptr(step.state_slot),
        out.data_ptr() + out_col0 * out.element_size(), _c_int(out.dtype == torch.float32 and x.dtype != torch.float32),
        _c_ll(out.stride(0)), _c_int(channels), _c_int(group), _c_int(n),
        _c_float(-1.0 if unit_eps is None else unit_eps), _c_int(scaled_groups), _c_float(group_scale),
        _c_int(int(move_state)), _c_int(CONV_ACTS[act])))
    return out


def conv_moves_state(step) -> bool:
    """Whether ``causal_conv`` may move the convolutions' state on itself in this step: every request brings one token."""
    return step.max_portion == 1


def conv_state_update(x: torch.Tensor, col0: int, channels: int, taps: int, slots: torch.Tensor, state_off: int,
                      step) -> None:
    """The convolution's state of every request of the step becomes the last ``taps - 1`` inputs it has seen."""
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and 0 <= col0 and col0 + channels <= x.shape[1],
          "conv_state_update: channels outside the rows")
    stride = _state_args(slots, "conv_state_update")
    _need(0 <= state_off and state_off + (taps - 1) * channels <= slots.shape[1],
          "conv_state_update: the state lies outside the slot")
    _check(library().rv_conv_state_update(
        _stream(), x.data_ptr() + col0 * x.element_size(), _dt(x), _c_ll(x.stride(0)), _c_int(taps), _ptr(slots),
        _c_ll(stride), _c_ll(state_off), _c_int(channels), _ptr(step.q_start), _ptr(step.state_slot), _c_int(channels),
        _c_int(step.num_requests)))


def delta_rule(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, ab: torch.Tensor, a_col: int, b_col: int,
               A_log: torch.Tensor, dt_bias: torch.Tensor, slots: torch.Tensor, state_off: int, step, heads: int,
               kv_heads: int, dk: int, dv: int) -> torch.Tensor:
    """The gated delta rule over the step's tokens, request by request in order.  ``qkv`` float32 rows: unit
    queries (scaled) and keys of ``kv_heads`` heads of ``dk``, values of ``heads`` heads of ``dv``, at their
    offsets; ``ab`` rows hold the decay's input of head h at ``a_col + h`` and beta's at ``b_col + h``;
    g = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b).  Per head S (32-bit, in the request's
    slot from ``state_off``, stored ``[heads, dv, dk]``: a column's dk numbers side by side): S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns o as
    float32 ``[tokens, heads * dv]``."""
    _gpu(qkv, A_log, dt_bias)
    n = qkv.shape[0]
    _need(qkv.dtype == torch.float32 and qkv.dim() == 2 and n == step.num_tokens, "delta_rule: float32 rows of the step's tokens")
    _need(ab.is_cuda and ab.dim() == 2 and ab.stride(1) == 1 and ab.shape[0] == n and ab.dtype in _DT
          and 0 <= a_col and a_col + heads <= ab.shape[1] and 0 <= b_col and b_col + heads <= ab.shape[1],
          "delta_rule: the gates' inputs lie outside their rows")
    _need(heads % kv_heads == 0 and max(q_off, k_off) + kv_heads * dk <= qkv.shape[1] and v_off + heads * dv <= qkv.shape[1],
          "delta_rule: heads outside the rows")
    _need(A_log.shape == (heads,) and dt_bias.shape == (heads,) and A_log.dtype == torch.float32
          and dt_bias.dtype == torch.float32, "delta_rule: float32 A_log and dt_bias, one a head")
    stride = _state_args(slots, "delta_rule")
    _need(0 <= state_off and state_off + heads * dk * dv <= slots.shape[1], "delta_rule: the state lies outside the slot")
    out = torch.empty((n, heads * dv), dtype=torch.float32, device=qkv.device)
    _check(library().rv_delta_rule(
        _stream(), _ptr(qkv), _c_ll(qkv.stride(0)), _c_int(q_off), _c_int(k_off), _c_int(v_off), _ptr(ab), _dt(ab),
        _c_ll(ab.stride(0)), _c_int(a_col), _c_int(b_col), _ptr(A_log), _ptr(dt_bias), _ptr(slots), _c_ll(stride),
        _c_ll(state_off), _ptr(step.q_start), _ptr(step.state_slot), _ptr(out), _c_int(step.num_requests), _c_int(heads),
        _c_int(kv_heads), _c_int(dk), _c_int(dv), _c_int(step.max_portion)))
    return out


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, gate_col0: int, weight: torch.Tensor, eps: float, heads: int,
                   dv: int, out_dtype: torch.dtype, act: str = "silu", divisor=None) -> torch.Tensor:
    """out[t, h] = o[t, h] / rms(o[t, h]) * weight * act(gate[t, gate_col0 + h dv ...]) for every head; ``weight`` is
    ``[dv]``, shared by the heads, or ``[heads * dv]``, every head its own; ``act`` is ``silu`` or ``sigmoid``.
    ``divisor`` = (dots float32 ``[tokens, heads]``, gates float32 ``[tokens, heads, 3]``): every head's o is first
    divided by max(|dot|, gates[..., 2]) + 1e-6 (what ``matrix_memory`` leaves undivided)."""
    _gpu(o, weight)
    n = o.shape[0]
    _need(o.dtype == torch.float32 and o.shape == (n, heads * dv), "head_norm_gate: float32 [tokens, heads * dv]")
    _need(weight.shape in ((dv,), (heads * dv,)) and weight.dtype == torch.float32,
          "head_norm_gate: a float32 weight of the head's size, or of all heads' size")
    _need(act in GATE_ACTS, f"head_norm_gate: unknown activation {act!r}")
    per_head = int(weight.shape[0] != dv)
    _need(gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and gate.dtype == out_dtype and gate.shape[0] == n
          and 0 <= gate_col0 and gate_col0 + heads * dv <= gate.shape[1], "head_norm_gate: the gate lies outside its rows")
    out = torch.empty((n, heads * dv), dtype=out_dtype, device=o.device)
    dots = floors = None
    if divisor is not None:
        dots, gates = divisor
        _gpu(dots, gates)
        _need(dots.shape == (n, heads) and gates.shape == (n, heads, 3) and dots.dtype == gates.dtype == torch.float32
              and dots.is_contiguous() and gates.is_contiguous(), "head_norm_gate: float32 dots [tokens, heads] and gates")
        floors = gates.data_ptr() + 2 * gates.element_size()
    _check(library().rv_head_norm_gate(_stream(), _ptr(o), gate.data_ptr() + gate_col0 * gate.element_size(),
                                       _c_ll(gate.stride(0)), _ptr(weight), _ptr(out), _dt(out), _c_int(n), _c_int(heads),
                                       _c_int(dv), _c_float(eps), _c_int(per_head), _c_int(GATE_ACTS[act]), _ptr(dots),
                                       floors, _c_int(3)))
    return out


def selective_scan(x: torch.Tensor, z: torch.Tensor, z_col0: int, dt: torch.Tensor, dt_bias: torch.Tensor,
                   bc: torch.Tensor, b_col: int, c_col: int, A_log: torch.Tensor, D: torch.Tensor, slots: torch.Tensor,
                   state_off: int, step) -> torch.Tensor:
    """The selective scan over the step's tokens, request by request in order.  ``x [tokens, channels]`` the
    convolved input, ``z`` the gate's input at ``z_col0`` of its rows, ``dt [tokens, channels]`` the step's
    projection (step = softplus(dt + dt_bias)), ``bc`` rows with B at ``b_col`` and C at ``c_col`` (``n`` each),
    A = -exp(A_log [channels, n]), D [channels].  S [channels, n] (32-bit, in the request's slot from
    ``state_off``): S <- exp(step A) S + step x B; y = S . C + D x.  Returns y * silu(z) in the type of ``x``."""
    _gpu(x, dt, dt_bias, A_log, D)
    n, channels = x.shape
    n_state = A_log.shape[1]
    _need(n == step.num_tokens and x.dtype in _DT, "selective_scan: the rows must be the step's tokens")
    _need(dt.shape == (n, channels) and dt.dtype == x.dtype, "selective_scan: bad dt")
    _need(z.is_cuda and z.dim() == 2 and z.stride(1) == 1 and z.dtype == x.dtype and z.shape[0] == n
          and 0 <= z_col0 and z_col0 + channels <= z.shape[1], "selective_scan: the gate lies outside its rows")
    _need(bc.is_cuda and bc.dim() == 2 and bc.stride(1) == 1 and bc.dtype == x.dtype and bc.shape[0] == n
          and 0 <= b_col and b_col + n_state <= bc.shape[1] and 0 <= c_col and c_col + n_state <= bc.shape[1],
          "selective_scan: B and C lie outside their rows")
    _need(A_log.shape == (channels, n_state) and D.shape == (channels,) and dt_bias.shape == (channels,)
          and A_log.dtype == D.dtype == dt_bias.dtype == torch.float32, "selective_scan: float32 A_log, D and dt_bias")
    stride = _state_args(slots, "selective_scan")
    _need(0 <= state_off and state_off + channels * n_state <= slots.shape[1], "selective_scan: the state lies outside the slot")
    out = torch.empty_like(x)
    _check(library().rv_selective_scan(
        _stream(), _ptr(x), _c_ll(x.stride(0)), z.data_ptr() + z_col0 * z.element_size(), _c_ll(z.stride(0)), _ptr(dt),
        _c_ll(dt.stride(0)), _ptr(dt_bias), _ptr(bc), _c_ll(bc.stride(0)), _c_int(b_col), _c_int(c_col), _ptr(A_log),
        _ptr(D), _ptr(slots), _c_ll(stride), _c_ll(state_off), _ptr(step.q_start), _ptr(step.state_slot), _ptr(out),
        _dt(x), _c_int(step.num_requests), _c_int(channels), _c_int(n_state), _c_int(step.max_portion)))
    return out


# ---- layer norm, and a residual stream kept in several copies -----------------------------------------------------
def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out_dtype: torch.dtype,
              rows: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(x - mean) / sqrt(variance + eps) * weight + bias over the last dimension, in 32-bit; ``x`` is 32-bit or of
    ``out_dtype``.  With ``rows`` (int32) the rows ``x[rows]``."""
    _gpu(x, weight, bias, rows, out)
    _need(x.dim() == 2 and x.is_contiguous() and x.dtype in _DT, "layernorm: a contiguous matrix expected")
    width = x.shape[1]
    _need(weight.shape == (width,) and bias.shape == (width,) and weight.dtype == bias.dtype and weight.dtype in _DT,
          "layernorm: a weight and a bias of the row's width and of one type")
    n = x.shape[0]
    if rows is not None:
        _i32(rows)
        n = rows.numel()
    if out is None:
        out = torch.empty((n, width), dtype=out_dtype, device=x.device)
    _need(out.shape == (n, width) and out.dtype == out_dtype and out.is_contiguous(), "layernorm: bad out")
    _check(library().rv_layernorm(_stream(), _ptr(x), _dt(x), _ptr(rows), _ptr(weight), _ptr(bias),
                                  _c_int(weight.dtype == torch.float32), _ptr(out), _dt(out), _c_int(n), _c_int(width),
                                  _c_float(eps)))
    return out


def streams_update(streams: torch.Tensor, out_dtype: torch.dtype, *, seed: Optional[torch.Tensor] = None, branch=None,
                   layer_scale: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                   out_w: Optional[torch.Tensor] = None, mult: float = 1.0, in_w: Optional[torch.Tensor] = None,
                   norm_w: Optional[torch.Tensor] = None, norm_b: Optional[torch.Tensor] = None, eps: float = 0.0,
                   total: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One sublayer's turn on the ``streams [S, tokens, width]`` (32-bit, in place) of a model that keeps S copies of
    its residual stream.  With ``seed`` all copies are first set to it.  With ``branch`` (the sublayer's result: a
    tensor of ``out_dtype``, ``SlicedSums`` or a ``BranchSum``), all streams at once from the old ones:
    x_t <- sum_s mix[s, t] x_s + mult * out_w[t] * (layer_scale * branch).  With ``in_w`` returns
    layernorm(sum_s in_w[s] x_s) of the streams as they then are, in ``out_dtype``: the next sublayer's input.
    With ``total`` (32-bit ``[tokens, width]``) the sum of the streams is written there."""
    _gpu(streams, seed, layer_scale, mix, out_w, in_w, norm_w, norm_b, total)
    _need(streams.dim() == 3 and streams.dtype == torch.float32 and streams.is_contiguous(),
          "streams_update: contiguous 32-bit streams [S, tokens, width]")
    S, n, width = streams.shape
    second, wa, wb = None, 1.0, 0.0
    if isinstance(branch, BranchSum):
        branch, second, wa, wb = branch.x, branch.y, branch.a, branch.b
    bptr, slices, stride, sptr, s_slices, s_stride = None, 0, 0, None, 0, 0
    if branch is not None:
        bptr, slices, stride, rows, b_width, bdtype = _branch_args(branch, "streams_update")
        _need((rows, b_width, bdtype) == (n, width, out_dtype), "streams_update: the branch must match the streams")
        if not isinstance(branch, SlicedSums):
            _need(branch.is_contiguous(), "streams_update: a contiguous branch")
        _need(mix is not None and out_w is not None and mix.shape == (S, S) and out_w.shape == (S,)
              and mix.dtype == out_w.dtype == torch.float32 and mix.is_contiguous(),
              "streams_update: 32-bit weights [S, S] and [S] go with a branch")
        if second is not None:
            sptr, s_slices, s_stride, s_rows, s_width, s_dtype = _branch_args(second, "streams_update")
            _need((s_rows, s_width, s_dtype) == (n, width, out_dtype), "streams_update: two branches of one shape and type")
    _need(seed is None or (seed.shape == (n, width) and seed.dtype == torch.float32 and seed.is_contiguous()),
          "streams_update: a 32-bit seed of a stream's shape")
    _need(layer_scale is None or (layer_scale.shape == (width,) and layer_scale.dtype == torch.float32),
          "streams_update: a 32-bit layer scale of the row's width")
    _need(total is None or (total.shape == (n, width) and total.dtype == torch.float32 and total.is_contiguous()),
          "streams_update: a 32-bit total of a stream's shape")
    nxt = None
    if in_w is not None:
        _need(in_w.shape == (S,) and in_w.dtype == torch.float32, "streams_update: 32-bit input weights [S]")
        _need(norm_w is not None and norm_b is not None and norm_w.shape == (width,) and norm_b.shape == (width,)
              and norm_w.dtype == norm_b.dtype and norm_w.dtype in _DT, "streams_update: the next norm's weight and bias")
        nxt = torch.empty((n, width), dtype=out_dtype, device=streams.device)
    _check(library().rv_streams_update(
        _stream(), _ptr(streams), _c_ll(n * width), _ptr(seed), bptr, _c_int(slices), _c_ll(stride), sptr,
        _c_int(s_slices), _c_ll(s_stride), _c_float(wa), _c_float(wb), _ptr(layer_scale), _ptr(mix), _ptr(out_w),
        _c_float(mult), _ptr(in_w), _ptr(norm_w), _ptr(norm_b),
        _c_int(norm_w is not None and norm_w.dtype == torch.float32), _ptr(nxt), _ptr(total), _DT[out_dtype], _c_int(S),
        _c_int(n), _c_int(width), _c_float(eps)))
    return nxt


# ---- a matrix memory with log gates; a gated linear recurrent unit -----------------------------------------------
def matrix_memory(rows: torch.Tensor, q_col: int, k_col: int, v_col: int, i_col: int, f_col: int, i_bias: torch.Tensor,
                  f_bias: torch.Tensor, cap: float, q_scale: float, slots: torch.Tensor, s_off: int, n_off: int,
                  m_off: int, step, heads: int, dk: int, dv: int) -> tuple[torch.Tensor, tuple]:
    """The matrix memory over the step's tokens, request by request in order.  The rows hold, head after head,
    queries at ``q_col`` and keys at ``k_col`` (``dk`` a head), values at ``v_col`` (``dv`` a head) and the two
    gates' inputs at ``i_col + h`` and ``f_col + h``.  Log gates i = cap tanh((a_i + i_bias) / cap),
    f = logsigmoid(cap tanh((a_f + f_bias) / cap)); m' = max(f + m, i); S' = e^(f + m - m') S + e^(i - m') k v^T, n
    likewise with k alone; o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6), q times ``q_scale``.  In the request's
    32-bit slot S lies at ``s_off`` as ``[heads, dv, dk]``, n at ``n_off`` ``[heads, dk]``, m at ``m_off`` ``[heads]``.
    Returns (S'^T q as float32 ``[tokens, heads * dv]``, not yet divided; the divisor's parts (n' . q ``[tokens,
    heads]``, gates ``[tokens, heads, 3]`` whose last entry is e^(-m'))): ``head_norm_gate(..., divisor=)`` divides."""
    _gpu(i_bias, f_bias)
    n = rows.shape[0]
    _need(rows.is_cuda and rows.dim() == 2 and rows.stride(1) == 1 and rows.dtype in _DT and n == step.num_tokens,
          "matrix_memory: rows of the step's tokens")
    width = rows.shape[1]
    _need(min(q_col, k_col, v_col, i_col, f_col) >= 0 and max(q_col, k_col) + heads * dk <= width
          and v_col + heads * dv <= width and max(i_col, f_col) + heads <= width, "matrix_memory: heads outside the rows")
    _need(i_bias.shape == (heads,) and f_bias.shape == (heads,) and i_bias.dtype == f_bias.dtype == torch.float32,
          "matrix_memory: float32 gate biases, one a head")
    stride = _state_args(slots, "matrix_memory")
    size = slots.shape[1]
    _need(0 <= s_off and s_off + heads * dk * dv <= size and 0 <= n_off and n_off + heads * dk <= size
          and 0 <= m_off and m_off + heads <= size, "matrix_memory: the state lies outside the slot")
    gates = torch.empty((n, heads, 3), dtype=torch.float32, device=rows.device)
    dots = torch.empty((n, heads), dtype=torch.float32, device=rows.device)
    out = torch.empty((n, heads * dv), dtype=torch.float32, device=rows.device)
    lib = library()
    _check(lib.rv_memory_gates(
        _stream(), _ptr(rows), _dt(rows), _c_ll(rows.stride(0)), _c_int(i_col), _c_int(f_col), _ptr(i_bias),
        _ptr(f_bias), _c_float(cap), _ptr(slots), _c_ll(stride), _c_ll(m_off), _ptr(step.q_start),
        _ptr(step.state_slot), _ptr(gates), _c_int(step.num_requests), _c_int(heads)))
    _check(lib.rv_memory_matrix(
        _stream(), _ptr(rows), _dt(rows), _c_ll(rows.stride(0)), _c_int(q_col), _c_int(k_col), _c_int(v_col),
        _c_float(q_scale), _ptr(gates), _ptr(slots), _c_ll(stride), _c_ll(s_off), _c_ll(n_off), _ptr(step.q_start),
        _ptr(step.state_slot), _ptr(out), _ptr(dots), _c_int(step.num_requests), _c_int(heads), _c_int(dk), _c_int(dv),
        _c_int(step.max_portion)))
    return out, (dots, gates)


GATED_SCAN_FEW = 4  # tokens a request up to which the recurrent unit's walk works its terms out itself


def gated_linear_scan(u: torch.Tensor, gates: torch.Tensor, block: int, r_bias: torch.Tensor, i_bias: torch.Tensor,
                      lam: torch.Tensor, y: torch.Tensor, y_col0: int, slots: torch.Tensor, s_off: int,
                      step) -> torch.Tensor:
    """The gated linear recurrent unit over the step's tokens, request by request in order, a channel at a time:
    r = sigmoid(g_r + r_bias), i = sigmoid(g_i + i_bias), log a = -8 r softplus(lam), S' = a S + sqrt(1 - a^2) i u,
    out = S' * gelu_tanh(y).  ``u [tokens, channels]`` is the convolved input, ``gates`` float32
    ``[tokens, 2 channels]`` holds for block b of ``block`` channels its g_r and then its g_i, ``y`` the other
    branch before its activation at ``y_col0`` of its rows.  S is 32-bit at ``s_off`` of the request's slot."""
    _gpu(u, gates, r_bias, i_bias, lam)
    n, channels = u.shape
    _need(n == step.num_tokens and u.dtype in _DT and u.stride(1) == 1, "gated_linear_scan: rows of the step's tokens")
    _need(gates.shape == (n, 2 * channels) and gates.dtype == torch.float32 and gates.stride(1) == 1,
          "gated_linear_scan: float32 gates [tokens, 2 channels]")
    _need(channels % block == 0, "gated_linear_scan: blocks of equal size")
    for t in (r_bias, i_bias, lam):
        _need(t.shape == (channels,) and t.dtype == torch.float32, "gated_linear_scan: float32 biases and rates, one a channel")
    _need(y.is_cuda and y.dim() == 2 and y.stride(1) == 1 and y.dtype == u.dtype and y.shape[0] == n
          and 0 <= y_col0 and y_col0 + channels <= y.shape[1], "gated_linear_scan: the other branch lies outside its rows")
    stride = _state_args(slots, "gated_linear_scan")
    _need(0 <= s_off and s_off + channels <= slots.shape[1], "gated_linear_scan: the state lies outside the slot")
    out = torch.empty((n, channels), dtype=u.dtype, device=u.device)
    terms = act = None
    if step.max_portion > GATED_SCAN_FEW:  # prompts: every token's terms by one launch, then the walk alone
        terms = torch.empty((2, n, channels), dtype=torch.float32, device=u.device)
        act = torch.empty((n, channels), dtype=u.dtype, device=u.device)
    _check(library().rv_gated_linear_scan(
        _stream(), _ptr(u), _c_ll(u.stride(0)), _ptr(gates), _c_ll(gates.stride(0)), _c_int(block), _ptr(r_bias),
        _ptr(i_bias), _ptr(lam), y.data_ptr() + y_col0 * y.element_size(), _c_ll(y.stride(0)), _ptr(slots),
        _c_ll(stride), _c_ll(s_off), _ptr(step.q_start), _ptr(step.state_slot), _ptr(out), _dt(u),
        _c_int(step.num_requests), _c_int(n), _c_int(channels), _ptr(terms), _ptr(act)))
    return out


def gemm_blocks_f32(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """A block-diagonal product with 32-bit results: ``w`` is ``[blocks, N, K]``; block b multiplies columns
    ``b K .. + K`` of the rows of ``a`` and fills columns ``b N .. + N`` of the float32 ``[rows, blocks N]``."""
    _need(a.is_cuda and w.is_cuda and a.dim() == 2 and w.dim() == 3 and w.is_contiguous() and a.stride(1) == 1
          and a.dtype == w.dtype and a.dtype in _DT, "gemm_blocks_f32: rows and [blocks, N, K] matrices of one type")
    blocks, n, k = w.shape
    m = a.shape[0]
    _need(blocks * k == a.shape[1], "gemm_blocks_f32: the blocks' inputs fill the rows")
    out = torch.empty((m, blocks * n), dtype=torch.float32, device=a.device)
    if a.dtype == torch.bfloat16 and _mfma_groups_take(a.data_ptr(), a.stride(0), w, k):  # on the matrix cores
        _check(library().rv_gemm_groups_mfma(
            _stream(), _ptr(a), _ptr(w), _ptr(out), None, None, _c_int(blocks), _c_int(m), _c_int(n), _c_int(k),
            _c_ll(a.stride(0)), _c_ll(k), _c_ll(out.stride(0)), _c_ll(k), _c_ll(n * k), _c_ll(n), None, _c_ll(0),
            _c_int(0), _c_float(0.0), _c_float(0.0), _c_int(1 if m <= MFMA_GROUPS_FEW_ROWS else 4), _c_int(1)))
        return out
    _check(library().rv_gemm_groups_plain(
        _stream(), _ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), None, None, _c_int(blocks), _c_int(m),
        _c_int(n), _c_int(k), _c_ll(a.stride(0)), _c_ll(k), _c_ll(out.stride(0)), _c_ll(k), _c_ll(n * k), _c_ll(n),
        None, _c_ll(0)))
    return out


# ---- experts chosen by a learned router ---------------------------------------------------------------------------
MOE_MAX_EXPERTS_TOPK = 1024


def moe_topk(logits: torch.Tensor, top: int) -> tuple[torch.Tensor, torch.Tensor]:
    """For every row of the float32 router logits ``[tokens, experts]`` its ``top`` largest (the largest first; of
    equal ones the lower index): (chosen int32 ``[tokens, top]``, weights float32 ``[tokens, top]`` =
    sigmoid(logit))."""
    _gpu(logits)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.is_contiguous(), "moe_topk: float32 logits")
    n, experts = logits.shape
    _need(1 <= top <= experts, f"moe_topk: {top} of {experts} experts")
    chosen = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=logits.device)
    _check(library().rv_moe_topk(_stream(), _ptr(logits), _c_int(n), _c_int(experts), _c_int(top), _ptr(chosen),
                                 _ptr(weights)))
    return chosen, weights


def moe_scale_rows(x: torch.Tensor, slot_of: torch.Tensor, weights: torch.Tensor, top: int, capacity: int) -> torch.Tensor:
    """The sorted rows of the experts' first product where a choice's weight multiplies the expert's input:
    xs[slot_of[t * top + k]] = weights[t, k] * x[t]; filling rows are zeros."""
    _gpu(x, slot_of, weights)
    _i32(slot_of)
    n, width = x.shape
    _need(x.is_contiguous() and x.dtype in _DT and slot_of.numel() == n * top and weights.numel() == n * top
          and weights.dtype == torch.float32, "moe_scale_rows: one weight and one sorted row for every choice")
    xs = torch.zeros((capacity, width), dtype=x.dtype, device=x.device)
    _check(library().rv_moe_scale_rows(_stream(), _ptr(x), _ptr(slot_of), _ptr(weights), _c_int(top), _ptr(xs), _dt(x),
                                       _c_int(n), _c_int(width)))
    return xs
