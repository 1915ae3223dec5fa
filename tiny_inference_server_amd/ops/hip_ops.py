"""The kernels as Python calls on torch tensors: what the parts and the engine compute with.

Every method checks on the host that shapes, dtypes and strides are what the kernel and its grid assume,
then launches on torch's current stream. There is no CPU path: without a GPU or without the compiled
libraries construction fails. Matrix products in bfloat16 of a few rows go to the fused few-row kernel
(csrc/gemm_skinny.hip), those of many rows to hipBLASLt through csrc/gemm_library.hip, as the reference's go to
a library (main_models_new.py:19-20); in 32-bit they go to the plain multiply-add kernel so that no
reduced-precision matrix mode can take part.

The library is only ever asked for products whose widths (output columns, input columns) stand in
ops/library_widths.json, the list of widths that this repository's GPU tests and benchmarks run, and only at row
counts from one family (library_rows): a library kernel differs from shape to shape, and a shape that nothing has
run is a kernel that nothing has tested. Any other product runs on this repository's own kernels: right at every
size, slower where there are many rows.
"""
from __future__ import annotations

import ctypes
import json
import os
from ctypes import c_float, c_int, c_long, c_void_p
from typing import NamedTuple, Optional

import numpy as np
import torch

from . import build as _build

_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _ptr(t: Optional[torch.Tensor]):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


class _Lib:
    """One compiled library with typed entry points that raise on failure."""

    def __init__(self, name: str, prefix: str, signatures: dict):
        self.name = name
        self.cdll = _build.load(name)
        self._err = getattr(self.cdll, f"{prefix}_last_error")
        self._err.restype = ctypes.c_char_p
        for fn, argtypes in signatures.items():
            f = getattr(self.cdll, fn)
            f.argtypes = argtypes
            f.restype = c_int
            setattr(self, fn, self._wrap(f))

    def _wrap(self, f):
        def call(*args):
            if f(*args) != 0:
                raise KernelError(self._err().decode(errors="replace"))
        return call


_P, _I, _L, _F = c_void_p, c_int, c_long, c_float

_SIGNATURES = {
    "rowwise": ("tis_rowwise", {
        "tis_rmsnorm": [_I, _P, _L, _P, _P, _L, _I, _I, _F, _P],
        "tis_embedding": [_I, _P, _P, _P, _L, _I, _I, _P],
        "tis_embedding_rmsnorm": [_I, _P, _P, _P, _P, _L, _I, _I, _F, _P],
        "tis_gather_rows": [_I, _P, _L, _P, _L, _P, _P, _L, _I, _I, _P],
        "tis_copy_rows": [_I, _P, _L, _P, _P, _L, _P, _I, _I, _P],
        "tis_swiglu": [_I, _P, _L, _P, _L, _I, _I, _P],
    }),
    "rope_cache": ("tis_rope_cache", {
        "tis_rope_write_kv": [_I, _P, _L, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _L, _P],
    }),
    "attention_generic": ("tis_attention_generic", {
        "tis_attention_generic": [_I, _P, _L, _P, _P, _I, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _F, _P, _P],
    }),
    "gemm_plain": ("tis_gemm_plain", {
        "tis_gemm_plain": [_I, _I, _P, _L, _P, _L, _P, _L, _P, _L, _I, _I, _I, _P],
    }),
    "sampling": ("tis_sampling", {
        "tis_sample": [_P, _L, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P],
        "tis_argmax": [_P, _L, _I, _I, _P, _P],
    }),
}

_SIGNATURES["gemm_skinny"] = ("tis_gemm_skinny", {
    "tis_gemm_skinny": [_P, _L, _P, _P, _F, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P],
    "tis_gemm_skinny_qkv_rope": [_P, _L, _P, _P, _F, _P, _L, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
})
_SIGNATURES["gemm_tiles"] = ("tis_gemm_tiles", {
    "tis_gemm_tiles": [_P, _L, _P, _P, _L, _P, _L, _I, _I, _I, _I, _P],
})
_SIGNATURES["gemm_library"] = ("tis_gemm_library", {
    "tis_gemm_library_init": [],
    "tis_gemm_library": [_P, _L, _P, _P, _L, _P, _L, _I, _I, _I, _I, _P],
})
_SIGNATURES["attention_mfma"] = ("tis_attention_mfma", {
    "tis_attention_mfma_side_stream": [_P],
    "tis_attention_mfma": [_P, _L, _P, _P, _I, _P, _P, _P, _I, _I, _P, _I, _P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _F,
                           _I, _I, _I, _I, _P, _P],
    "tis_attention_mfma_sink": [_P, _L, _P, _P, _I, _P, _P, _P, _I, _I, _P, _I, _P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _F,
                                _I, _I, _I, _I, _P, _I, _P],
})

_SIGNATURES["stream32"] = ("tis_stream32", {
    "tis_embed_scale": [_I, _P, _P, _F, _P, _P, _I, _I, _P],
    "tis_gated_postnorm": [_I, _P, _P, _L, _F, _P, _L, _F, _P, _L, _P, _F, _P, _F, _P, _P, _I, _I, _P],
    "tis_rmsnorm32": [_I, _P, _P, _F, _P, _L, _I, _I, _P],
    "tis_head_norm_gate": [_I, _P, _L, _P, _L, _P, _I, _I, _F, _P, _L, _I, _I, _I, _P],
    "tis_lowrank_decay": [_P, _L, _I, _P, _P, _F, _P, _I, _I, _P],
    "tis_layernorm32": [_I, _P, _P, _P, _F, _P, _L, _I, _I, _P],
    "tis_residual_norm": [_I, _P, _P, _L, _P, _F, _P, _P, _L, _I, _P, _P, _F, _P, _L, _I, _I, _P, _P, _I, _I, _P, _L, _P, _L,
                          _P, _L, _P],
    "tis_gate_table": [_I, _P, _L, _P, _L, _P, _I, _P, _L, _I, _I, _P],
    "tis_activate32": [_P, _L, _I, _I, _I, _P],
    "tis_head_gate": [_I, _P, _L, _P, _L, _I, _I, _I, _P],
    "tis_dyt32": [_I, _P, _F, _P, _P, _P, _L, _I, _I, _P],
    "tis_scaled_sum": [_I, _P, _P, _L, _P, _P, _P, _L, _P, _P, _P, _P, _I, _I, _P, _L, _P, _I, _F, _P, _P, _P, _L, _I, _I,
                       _P],
    "tis_gated_act": [_I, _P, _L, _I, _P, _P, _P, _I, _P, _L, _I, _F, _P],
    "tis_softcap": [_P, _L, _F, _I, _I, _P],
    "tis_lowrank_act": [_P, _L, _I, _P, _P, _I, _F, _P, _I, _P, _I, _I, _P],
    "tis_normed_mean": [_P, _L, _P, _P, _L, _P, _F, _P, _I, _I, _P],
    "tis_activate_rows": [_I, _P, _L, _I, _P, _L, _I, _I, _P],
})
_SIGNATURES["attention_window"] = ("tis_attention_window", {
    "tis_attention_prepare": [_I, _P, _L, _I, _I, _I, _P, _P, _P, _P, _L, _P, _P, _P, _P, _P, _P, _P, _I, _F, _I, _F, _I,
                              _I, _I, _I, _I, _I, _I, _I, _I, _P],
    "tis_latent_prepare": [_I, _P, _L, _I, _I, _P, _P, _P, _P, _L, _P, _L, _P, _P, _I, _F, _I, _I, _I, _I, _I, _I, _P],
    "tis_attention_window": [_I, _P, _L, _P, _P, _I, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P, _L, _P],
    "tis_attention_mixed": [_I, _P, _L, _P, _P, _I, _P, _P, _P, _L, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _F, _P, _P, _I, _P],
})
_SIGNATURES["attention_latent"] = ("tis_attention_latent", {
    "tis_attention_latent": [_P, _L, _P, _P, _I, _P, _P, _P, _I, _P, _L, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
})
_SIGNATURES["experts"] = ("tis_experts", {
    "tis_route_topk": [_P, _L, _P, _F, _I, _I, _I, _I, _P, _P, _I, _I, _I, _P],
    "tis_expert_lists": [_P, _I, _I, _I, _P, _P, _P],
    "tis_grouped_linear": [_I, _I, _P, _L, _L, _I, _P, _P, _L, _L, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "tis_experts_combine": [_I, _P, _L, _P, _L, _P, _P, _I, _I, _P, _L, _I, _I, _P],
})
_SIGNATURES["state_scan"] = ("tis_state_scan", {
    "tis_state_scan": [_I, _P, _L, _I, _I, _I, _F, _P, _L, _I, _I, _P, _P, _F, _P, _L, _P, _P, _I, _P, _L, _I, _I, _I, _I,
                       _I, _I, _P, _I, _I, _P],
})
_SIGNATURES["ssm_parts"] = ("tis_ssm", {
    "tis_conv_prepare": [_P, _L, _I, _I, _P, _P, _P, _P, _P, _L, _I, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P],
    "tis_conv_state_update": [_P, _L, _I, _P, _L, _I, _P, _P, _I, _I, _I, _P],
    "tis_gated_group_norm": [_I, _P, _L, _P, _L, _P, _I, _P, _L, _P, _F, _P, _L, _I, _I, _I, _P],
})

_SIGNATURES["delta_rule"] = ("tis_delta_rule", {
    "tis_delta_prepare": [_P, _L, _I, _I, _P, _I, _P, _L, _I, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P],
    "tis_delta_scan": [_P, _L, _I, _I, _I, _I, _P, _L, _P, _L, _P, _P, _I, _P, _L, _I, _I, _I, _I, _P],
})

_SIGNATURES["attention_mixed"] = ("tis_attention_mixed", {
    "tis_attention_mixed_mfma": [_P, _L, _P, _P, _I, _P, _P, _P, _I, _P, _L, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _F, _P, _P, _P],
})

_libs = {}


def library(name: str) -> _Lib:
    """`name` may carry a variant: 'attention_mfma@128'."""
    lib = _libs.get(name)
    if lib is None:
        prefix, sigs = _SIGNATURES[name.split("@")[0]]
        lib = _libs[name] = _Lib(name, prefix, sigs)
    return lib


_FEW_ROWS = 128                 # up to this many rows a product goes to the few-row kernels whatever its widths

_WIDTHS_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "library_widths.json")


def library_widths(path: str = _WIDTHS_FILE):
    """The (output columns, input columns) pairs that may go to the library's product: a data file, not code."""
    with open(path) as f:
        return frozenset((int(n), int(k)) for n, k in json.load(f)["widths"])


def library_rows(m: int) -> int:
    """The row count the library is asked for when a product has `m` rows: the next multiple of 64 up to 256 rows,
    of 256 beyond. A serving run's steps bring row counts that nobody chose (a portion beside some decoded tokens, a
    prediction head's rows one short of the trunk's); rounded up, they all become the few shapes that every
    benchmark and test of a width has already run. The extra rows are computed on whatever lies behind the operands'
    rows and are never read."""
    step = 64 if m <= 256 else 256
    return -(-m // step) * step


def product_route(M: int, N: int, K: int, aligned: bool, out_f32: bool, widths, few_rows: int = _FEW_ROWS):
    """Which kernel takes a bfloat16 product of M rows, N output and K input columns: "few_rows" (the fused few-row
    kernel, in panels of rows beyond its own height), "library" (at library_rows(M) rows, at the widths of its
    list), "tiles" (this repository's tiled product, for many rows at any other width and for 32-bit results at any
    width) or "plain" (multiply-adds, for operands that do not lie as the others need them). Pure: the decision can be checked without a device."""
    if not aligned:
        return "plain"
    if M <= few_rows:
        return "few_rows"
    if (N, K) in widths and not out_f32:
        return "library"
    return "tiles" if N % 4 == 0 else "few_rows"


# wavefronts the attention launch aims for, so that short batches still spread over the chip
_ATTN_TARGET_WAVES = 512
_CHIP_UNITS = 256               # compute units of an MI355X: the default where no device is asked (host-only tests)
_ATTN_PROMPT_TARGET_WAVES = 2048  # what the grid offers where rows of prompts are in the batch ...
_ATTN_PROMPT_SPLIT_MAX_ROWS = 512 # ... and the batch is small; a long portion fills the chip by its rows alone
_ATTN_PROMPT_MIN_STEPS = 8         # steps of 32 keys below which a prompt item's split is not worth its merge
_ATTN_UNEVEN = 1.5              # decoded tokens: from this ratio of the longest request to the mean on, splits are planned
                                # request by request on the host instead of being the same for all
_ATTN_DECODE_MAX_SPLITS = 64    # ... and the most that one request may get
_ATTN_PLANNED_MIN_ROWS = 16     # ... where there are at least this many requests (8: as fast either way) ...
_ATTN_PLANNED_MAX_WAVES = 384   # ... and requests x key/value heads are at most this: beyond, there are too few splits
                                # to shift between requests and the plain grid is as fast or faster. A planned list
                                # aims at one entry (a wave per key/value head) per compute unit, and at
                                # _ATTN_TARGET_WAVES waves at least. Uneven requests of 128 to 4,200 keys, planned /
                                # same splits for all, us: 3 kv heads, 96 requests 72 / 87, 64: 43 / 47, 24: 20.5 /
                                # 24.6; 4 heads, 96: 100 / 103, 48: 39 / 43; 8 heads, 64: 126 / 124, 32: 53.5 / 60.6;
                                # 1 head, 64: 19.8 / 21.0; with 8 requests 13.2 / 12.4 (3 heads), 23.6 / 21.8 (8)
_ATTN_DECODE_BYTES_PER_US = 5.0e6   # keys and values a step of decoded tokens streams: 5 TB/s
_ATTN_PLANNED_BESIDE_FROM = 1.15   # single rows beside tiles get a planned list if they take this much longer than the tiles
_ATTN_PLANNED_WAVES_BESIDE_TILES = 1.5   # ... and at this many waves per compute unit, over all key/value heads, where
                                # the list runs beside a portion's tiles, whose workgroups need room on every unit
_ATTN_MIN_SPLIT_KEYS = 128      # a split shorter than this costs more in merging than it gains in spreading
_ATTN_TILE_WAVES = 4            # waves of the workgroup that takes a tile of a long portion
_ATTN_TILE_GROUPS = 512         # workgroups of the tile kernel that the chip runs side by side
_ATTN_TILE_MIN_STEPS = 8        # steps of 32 keys below which a tile's split is not worth its merge
_ATTN_TILE_SPLIT_SLACK = 1.4    # a split may be this much longer than an even share of all steps
_ATTN_TILE_STEP_US = (0.72, 1.3)   # what a tile's step of 32 keys takes while a workgroup has a compute unit to itself,
                                # and once two share one (12 heads of 128 over 3; other geometries differ little)
_ATTN_TILE_MERGE_US = (10.0, 4.0, 6e6)   # what cutting tiles into key splits costs beyond the tiles' own time: the
                                # merge's launch and the per-row counts (less where the items' splits are merged anyway),
                                # and microseconds per byte of 32-bit partial results. Tiles are cut only where, by
                                # these figures, the shorter chains save more than that. 12 heads of 128 over 3, us,
                                # cut / uncut / one-wave kernel: 4 prompts of 512 tokens 28.8 / 18.8 / 22.8, 8 of 512
                                # 40.8 / 25.4 / 33.2, 4 of 1,024 50.6 / 39.5 / 57.2, one of 1,024 29.2 / 28.6 / 29.2; but
                                # one of 1,536 35.3 / 39.9 / 47.7, of 2,048 42.4 / 51.3 / 69.5, 512 tokens behind 3,000
                                # others 41.5 / 82.5 / 60.0
_ATTN_TILE_PARTIAL_BYTES = 40 << 20   # partial results (32-bit, per split) beyond which the merge costs more than
                                      # shorter chains save; at least two splits are always allowed
_ATTN_TILE_MIN_WORK_MIXED = 1500   # tile steps times key/value heads below which the one-wave kernel is the faster
                                   # beside decoded tokens deep in their requests (few tiles with long chains: the
                                   # one-wave kernel spreads them over more waves, and its splits are merged anyway)
_ATTN_WORKSPACE_FLOATS = 16 << 20


def tile_columns(head_dim: int) -> int:
    """Columns (row, query head of a group) of one wave of the tile kernel, as the kernel source sets them."""
    return 32


def attention_items(seq_rows, group_size: int, tile_cols: int = 0, n_kv_heads: int = 0):
    """Work items of the matrix-core attention kernels for the rows of one stage.

    seq_rows: (first row, first position, rows) per request. Returns (column blocks per item, items, tiles, steps):
    items and tiles are int32 arrays of (first row, rows) lines that together hold every row once, steps is
    (the number of 32-key steps that all tiles walk together, the most that one tile walks): the kernel's work, by
    which its key splits are sized.
    An item (one wave) holds consecutive rows of one request, rows * group_size <= 16 * blocks. When no request has
    more than one row the list is simply every row in order, which the kernel knows without being given a list.
    A tile (a workgroup of four waves, `tile_cols` columns each; 0: no tiles) takes up to 4 * (tile_cols // group_size)
    consecutive rows of a portion that fills at least half of one. Beside decoded tokens deep in their requests, tiles
    are made only where their steps times `n_kv_heads` (the workgroups' work; 0: always) reach
    _ATTN_TILE_MIN_WORK_MIXED. Measured at 12 heads of 128 over 3 (tiles / one-wave kernel, us): one prompt of 256
    rows 12.1 / 13.3, of 512 rows 17.5 / 22.3, of 1,024 rows 28.6 / 29.2, 8 of 512 rows 25.4 / 33.2; a portion of 512
    rows at 1,000 beside 8 decoded tokens at 4,095: 54.9 / 64.7, one of 256 rows 40.6 / 30.1, one of 128 35.9 / 23.9.
    """
    none = np.zeros((0, 2), dtype=np.int32)
    # (arrays over all requests at once: a step may hold hundreds, and this runs for every stage of every step that
    # is not replayed from a graph)
    rows = np.asarray(seq_rows, dtype=np.int64).reshape(-1, 3)
    first, p0, n = rows[:, 0], rows[:, 1], rows[:, 2]
    if not (n > 1).any():
        nb = 1
        while group_size > 16 * nb:
            nb *= 2
        live = n > 0
        return nb, np.stack((first[live], n[live]), axis=1).astype(np.int32), none, (0, 0)

    def cut(which, per_item):
        if not which.any():
            return none, (0, 0)
        f, q0, m = first[which], p0[which], n[which]
        k = -(-m // per_item)                                          # items of each segment
        r = (np.arange(int(k.sum())) - np.repeat(np.cumsum(k) - k, k)) * per_item    # an item's first row in its segment
        counts = np.minimum(per_item, np.repeat(m, k) - r)
        firsts = np.repeat(f, k) + r
        keys = np.repeat(q0, k) + r + counts
        # those with the most keys first: under a causal mask the last rows of a prompt are the longest, and
        # started last they would run on alone while the rest of the chip idles
        order = np.argsort(-keys, kind="stable")
        steps = (keys + 31) // 32
        return np.stack((firsts[order], counts[order]), axis=1).astype(np.int32), (int(steps.sum()), int(steps.max()))

    tile_rows = _ATTN_TILE_WAVES * (tile_cols // group_size)
    tiled = (n >= max(2, tile_rows // 2)) if tile_rows else np.zeros(len(n), dtype=bool)
    tiles, steps = cut(tiled, tile_rows) if tile_rows else (none, (0, 0))
    if len(tiles) and n_kv_heads and steps[0] * n_kv_heads < _ATTN_TILE_MIN_WORK_MIXED \
            and ((n == 1) & (p0 >= 512)).any():
        # beside decoded tokens deep in their requests: too little work for tiles
        tiled, tiles, steps = np.zeros(len(n), dtype=bool), none, (0, 0)
    rest = (n > 0) & ~tiled
    nb = 2
    # 64-column items halve what a portion reads of its keys and values; they pay once there are enough of them
    # to fill the chip, and cost where a few long chains of steps set the time
    if group_size <= 64 and int((-(-n[rest] // max(1, 64 // group_size))).sum()) >= 384:
        nb = 4
    while group_size > 16 * nb:
        nb *= 2
    return nb, cut(rest, max(1, (16 * nb) // group_size))[0], tiles, steps


def first_key(pos: int, window: int) -> int:
    """The first key that the row at position pos sees, as the matrix-core attention kernels count: window > 0: the
    last `window` keys; window < 0: the keys of the row's own chunk of -window positions, from the last multiple of
    that size on; 0: all."""
    if window > 0:
        return max(0, pos - window + 1)
    if window < 0:
        return pos - pos % (-window)
    return 0


def row_steps(pos: int, window: int) -> int:
    """32-key steps that a wave walks for the row at position pos: from a multiple of 32 to the row's own key."""
    return (pos + 32 - (first_key(pos, window) & ~31)) >> 5


def uneven_lengths(seq_rows, window: int = 0) -> bool:
    """Whether a step of single rows holds requests of such different lengths that equal split counts would leave the
    longest request's waves running on alone: then the splits are planned request by request (decode_items). With a
    window a row's length is what it sees of its request."""
    n = len(seq_rows)
    if n < 2:
        return False
    longest = total = 0
    for _, p0, rows in seq_rows:            # (one pass: this runs for every step of decoded tokens)
        if rows != 1:
            return False
        steps = row_steps(p0, window)
        total += steps
        if steps > longest:
            longest = steps
    return longest * n > _ATTN_UNEVEN * total + 2 * n


def planned_list_pays(n_rows: int, n_kv_heads: int) -> bool:
    """Whether single rows of uneven lengths get a planned list rather than the same splits for all."""
    return n_rows >= _ATTN_PLANNED_MIN_ROWS and n_rows * n_kv_heads <= _ATTN_PLANNED_MAX_WAVES


def planned_target_waves(n_kv_heads: int, units: int = _CHIP_UNITS) -> int:
    return max(_ATTN_TARGET_WAVES, units * n_kv_heads)


def decode_items_capacity(n_rows: int, n_kv_heads: int, units: int = _CHIP_UNITS) -> int:
    """Entries of a planned list for `n_rows` single rows: what the splits can add up to, whatever the lengths."""
    # (a multiple of the eight XCDs: workgroups go to them in turn, so the waves of an entry's key/value heads, which
    # read the same pages, then meet in one L2: 162 against 183 us at 8 key/value heads)
    return -(-(planned_target_waves(n_kv_heads, units) // n_kv_heads + n_rows + 1) // 8) * 8


def decode_items_most_splits(n_rows: int, n_heads: int, head_dim: int, workspace_floats=None) -> int:
    """The most splits one row of such a list may have: bounded by the workspace for partial results."""
    workspace_floats = _ATTN_WORKSPACE_FLOATS if workspace_floats is None else workspace_floats
    return int(max(1, min(_ATTN_DECODE_MAX_SPLITS, (workspace_floats - n_rows) // (n_rows * n_heads * (head_dim + 2)))))


def decode_items(seq_rows, n_heads: int, n_kv_heads: int, head_dim: int, workspace_floats=None, window: int = 0,
                 units: int = _CHIP_UNITS, table_lines=None, all_rows: int = 0, share: float = 1.0):
    """The work list of a step of single rows whose requests differ widely in length: one entry per wave (and
    key/value head), (row, split + 65536 * splits of the row, position, block-table line), so that every wave walks
    about the same number of keys; longest first; padded with row -1 to a length that depends on the number of rows
    alone (a captured launch keeps its grid while the lengths change). Returns (int32 [capacity, 4], most splits).
    table_lines: the rows' lines of the block table where they are not simply 0, 1, ... (single rows beside portions
    of other requests); all_rows: the rows of the whole step then (they share the workspace for partial results)."""
    n = len(seq_rows)
    rows = np.fromiter((f for f, _, _ in seq_rows), dtype=np.int64, count=n)
    pos = np.fromiter((p0 for _, p0, _ in seq_rows), dtype=np.int64, count=n)
    # a row at position p sees p + 1 keys, or the last `window` of them; the kernel walks them in steps of 32 from a
    # multiple of 32
    first = np.maximum(0, pos - window + 1) & ~31 if window > 0 else (pos - pos % (-window)) & ~31 if window < 0 else 0
    steps = (pos + 32 - first) // 32
    fewest = max(1, _ATTN_MIN_SPLIT_KEYS // 32)
    even = max(fewest, -(-int(steps.sum()) * n_kv_heads // max(1, int(planned_target_waves(n_kv_heads, units) * share))))
    most = decode_items_most_splits(max(n, all_rows), n_heads, head_dim, workspace_floats)
    splits = np.clip((steps + even // 2) // even, 1, np.minimum(steps, most))
    cap = decode_items_capacity(n, n_kv_heads, units)
    total = int(splits.sum())
    if total > cap:
        raise KernelError(f"attention: {total} planned splits for a list of {cap}")
    # one entry per (row, split); those with the most steps first, and among equals split by split over all rows, so
    # that waves that start together read different requests' pages (the order a grid of rows x splits would have)
    who = np.repeat(np.arange(n), splits)
    which = np.arange(total) - np.repeat(np.cumsum(splits) - splits, splits)
    per_split = -(-steps // splits)
    by = np.lexsort((who, which, -per_split[who]))
    who, which = who[by], which[by]
    out = np.full((cap, 4), -1, dtype=np.int32)
    out[:total, 0] = rows[who]
    out[:total, 1] = which + (splits[who] << 16)
    out[:total, 2] = pos[who]
    out[:total, 3] = who if table_lines is None else np.asarray(table_lines, dtype=np.int64)[who]
    return out, most


def planned_beside_tiles(seq_rows, items, tiles, tile_steps, n_heads: int, n_kv_heads: int, head_dim: int,
                         window: int = 0, units: int = _CHIP_UNITS):
    """For a step whose portions all go to tiles and whose other rows are single rows of requests that differ widely
    in length (decoded tokens beside a prompt's portion): the planned list of decode_items for those rows, or None.
    With the same number of splits for every row the longest request's waves would run on alone, here beside the
    tiles' workgroups. It pays where the single rows are the longer half of the pair: beside tiles that take as long as
    they do or longer (a portion deep in a long prompt) the rows are done first either way, and the list only costs the
    host its making. 64 decoded tokens at 512 to 8,000 keys, us a layer, planned / same splits for all, 12 heads over 3:
    beside a 2,048-token prompt 125 / 151, beside 1,024 tokens behind 1,000 others 126 / 151, beside 2,048 behind
    2,048 others 143 / 154; 16 over 4: 158 / 191, 164 / 195 and 197 / 186."""
    n_items = len(items)
    if not len(tiles) or n_items < _ATTN_PLANNED_MIN_ROWS or n_items * n_kv_heads > _ATTN_PLANNED_MAX_WAVES \
            or n_heads // n_kv_heads > 64 or int(items[:, 1].max()) != 1:
        return None
    singles, lines, all_rows = [], [], 0
    for i, (f, p0, n) in enumerate(seq_rows):
        all_rows += n
        if n == 1:
            singles.append((f, p0, 1))
            lines.append(i)
    if len(singles) != n_items or not uneven_lengths(singles, window):
        return None
    # what the rows take at the rate a step of decoded tokens streams keys and values, against the tiles' estimate
    steps_of_rows = sum(row_steps(p0, window) for _, p0, _ in singles)
    rows_us = steps_of_rows * n_kv_heads * 64 * head_dim * 2 / _ATTN_DECODE_BYTES_PER_US
    cut, cut_steps = _tiles_cut(all_rows, len(tiles), tile_steps, n_heads, n_kv_heads, head_dim)
    tiles_us = min(_tiles_us(all_rows, len(tiles), tile_steps[0], tile_steps[1], cut, cut_steps, n_heads, n_kv_heads,
                             head_dim, True, units))
    if rows_us < _ATTN_PLANNED_BESIDE_FROM * tiles_us:
        return None
    return decode_items(singles, n_heads, n_kv_heads, head_dim, window=window, units=units, table_lines=lines,
                        all_rows=all_rows, share=min(1.0, _ATTN_PLANNED_WAVES_BESIDE_TILES / n_kv_heads))


def latent_items(seq_rows, n_heads: int, columns: int = 64):
    """(first row, rows) of every item of the latent-attention kernel for portions: `columns` columns an item, a column a
    (row, head) pair, so columns // heads consecutive rows of one request where there are fewer heads than columns, a
    single row otherwise."""
    per = max(1, columns // n_heads)
    rows = np.asarray(seq_rows, dtype=np.int64).reshape(-1, 3)
    first, n = rows[:, 0], rows[:, 2]
    k = -(-n // per)
    r = (np.arange(int(k.sum())) - np.repeat(np.cumsum(k) - k, k)) * per
    counts = np.minimum(per, np.repeat(n, k) - r)
    return np.stack((np.repeat(first, k) + r, counts), axis=1).astype(np.int32)


class ChosenExperts(NamedTuple):
    """A routed feed-forward's result before the sum over a row's choices."""
    results: Optional[torch.Tensor]     # [rows * top, width] 32-bit, a line per (row, choice); None with no real expert
    ids: torch.Tensor                   # [rows, top] int32
    weights: torch.Tensor               # [rows, top] 32-bit
    n_experts: int                      # ids from here on are identity experts
    rows: torch.Tensor                  # [rows, width] in the compute type: what the feed-forward read
    extra: Optional[torch.Tensor] = None        # [rows, width] 32-bit: what every row adds beside its choices (a shared
    extra_gate: Optional[torch.Tensor] = None   # expert), times sigmoid(extra_gate [rows, 1] 32-bit, a strided view is fine)


class AttentionLaunch(NamedTuple):
    """How one call of the matrix-core attention cuts its keys, and where its partial results lie in the workspace
    (offsets in floats): [rows][heads][stride][head size] outputs, then [rows][heads][stride] (maximum, sum) pairs,
    then [rows] split counts."""
    n_splits: int
    min_steps: int
    tile_splits: int
    tile_max_steps: int
    stride: int
    ml_offset: int
    row_splits_offset: int
    need_floats: int


def _tiles_us(n, n_tiles, all_steps, longest, cut, cut_steps, n_heads, n_kv_heads, head_dim, merged_anyway, units):
    """Estimated microseconds of a call's tiles left whole, and cut into `cut` key splits of at most `cut_steps` steps:
    the longest chain of steps sets the time (a step takes longer once two workgroups share a compute unit, and no
    less than all steps spread evenly take), and the cut adds the merge."""
    alone, shared = _ATTN_TILE_STEP_US

    def chain_us(steps, workgroups):
        return max(steps * min(shared, alone * max(1.0, workgroups / units)), all_steps * n_kv_heads / (2 * units) * shared)
    whole = chain_us(longest, n_tiles * n_kv_heads)
    launch, launch_merged, bytes_per_us = _ATTN_TILE_MERGE_US
    merge = (launch_merged if merged_anyway else launch) + n * n_heads * head_dim * 4 * cut / bytes_per_us
    parts = chain_us(cut_steps, n_kv_heads * (all_steps / cut_steps + n_tiles / 2)) + merge
    return whole, parts


def _tiles_cut_pays(*args) -> bool:
    """Whether cutting the tiles of a call into key splits is estimated to be faster than leaving them whole."""
    whole, parts = _tiles_us(*args)
    return parts < whole


def _tiles_cut(n, n_tiles, tile_steps, n_heads, n_kv_heads, head_dim):
    """Into how many key splits, of at most how many steps, a call's tiles would be cut if they are cut."""
    all_steps, longest = tile_steps
    share = all_steps * n_kv_heads / _ATTN_TILE_GROUPS
    cut_steps = max(_ATTN_TILE_MIN_STEPS, int(share * _ATTN_TILE_SPLIT_SLACK) + 1)
    most_splits = max(2, _ATTN_TILE_PARTIAL_BYTES // (n * n_heads * head_dim * 4))
    cut = max(1, min(most_splits, -(-longest // cut_steps)))
    return cut, max(cut_steps, -(-longest // cut))


def attention_launch_plan(n, n_items, n_tiles, tile_steps, single, max_kv_len, n_heads, n_kv_heads, head_dim,
                          workspace_floats=None, planned_splits=0, units: int = _CHIP_UNITS) -> AttentionLaunch:
    """Split counts of one attention call over `n` rows, from the planner's items and tiles; pure host arithmetic.
    planned_splits > 0: the items are a list planned by decode_items, whose rows have at most that many splits."""
    workspace_floats = _ATTN_WORKSPACE_FLOATS if workspace_floats is None else workspace_floats
    n_splits, min_steps, tile_splits, tile_max_steps = 1, 0, 1, 1 << 20
    if planned_splits:
        n_splits, min_steps = planned_splits, -1
    elif n_items:
        # decoded tokens: every request's keys are cut into the same number of splits, enough to spread a
        # short batch over the chip. Prompt rows: the grid offers more splits than the chip needs and every
        # item takes as many as its own length deserves (the kernel decides, from _ATTN_PROMPT_MIN_STEPS),
        # because the last rows of a long prompt would otherwise run on alone long after the first have finished.
        target = _ATTN_PROMPT_TARGET_WAVES if (not single and n <= _ATTN_PROMPT_SPLIT_MAX_ROWS) else _ATTN_TARGET_WAVES
        # a lone request or two: shorter splits still pay, because so few waves would leave most of the chip idle
        min_keys = _ATTN_MIN_SPLIT_KEYS // 2 if n_items * n_kv_heads <= 8 else _ATTN_MIN_SPLIT_KEYS
        n_splits = max(1, min(-(-target // (n_items * n_kv_heads)), max_kv_len // min_keys))
        if single and n_splits > 1:
            # equal waves spread evenly only if their number is a whole multiple of the chip's compute units: a few
            # more splits that reach one beat the target's count (64 requests over 3 heads at 4,096 keys: 4 splits
            # 79 us, 3 splits 82; 32 requests: 8 splits 37, 6 splits 40; at 8,192 keys 146 against 163)
            waves = n_items * n_kv_heads
            for s in range(n_splits, min(2 * n_splits, max_kv_len // min_keys) + 1):
                if waves * s % units == 0:
                    n_splits = s
                    break
        min_steps = 0 if single else _ATTN_PROMPT_MIN_STEPS
    if n_tiles:
        # a tile's keys are cut so that no workgroup walks a chain of steps much longer than an even share of
        # all tiles' steps: the last rows of a long prompt would otherwise run on alone. Measured at 12 heads
        # of 128 (tiles / one-wave kernel, us): 2,048 rows from 0: 54 / 69; from 2,048: 99 / 134; from 6,144:
        # 196 / 260; 4,096 rows: 146 / 202.
        all_steps, longest = tile_steps
        cut, cut_steps = _tiles_cut(n, n_tiles, tile_steps, n_heads, n_kv_heads, head_dim)
        if cut > 1 and _tiles_cut_pays(n, n_tiles, all_steps, longest, cut, cut_steps, n_heads, n_kv_heads, head_dim,
                                       n_splits > 1, units):
            tile_splits, tile_max_steps = cut, cut_steps
    # partial results of split key ranges live in one workspace of fixed size; fewer splits where it
    # would not suffice
    most = max(1, (workspace_floats - n) // (n * n_heads * (head_dim + 2)))
    n_splits, tile_splits = min(n_splits, most), min(tile_splits, most)
    stride = max(n_splits, tile_splits)
    ml_offset = n * n_heads * stride * head_dim
    rs_offset = n * n_heads * stride * (head_dim + 2)
    return AttentionLaunch(n_splits, min_steps, tile_splits, tile_max_steps, stride, ml_offset, rs_offset,
                           rs_offset + n if stride > 1 else 0)


_side_streams = {}


def _side_stream(device_index: int):
    """The device's second stream (default priority), on which the attention library runs a step's tiles beside its
    items. One per device for the life of the process: the library keeps its handle."""
    s = _side_streams.get(device_index)
    if s is None:
        s = _side_streams[device_index] = torch.cuda.Stream(torch.device("cuda", device_index))
    return s


def _rows_view(t: torch.Tensor, what: str):
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what}: expected a 2-d tensor with unit column stride, got shape {tuple(t.shape)} "
                          f"strides {t.stride()}")
    return t


class HipOps:
    """The operations of one engine instance: a device, a compute dtype, and the kernels for them."""
    supports_graphs = True      # every launch goes to torch's current stream, so a stream capture records it

    def __init__(self, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in _DT:
            raise KernelError(f"unsupported compute dtype {dtype}; use torch.bfloat16 or torch.float32")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: this engine runs on HIP kernels only and has no CPU path")
        self.device = torch.device(device)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.dtype = dtype
        self.code = _DT[dtype]
        # whatever is not built yet is compiled side by side, not one after the other
        _build.build(["rowwise", "rope_cache", "attention_generic", "gemm_plain", "sampling"] +
                     (["gemm_skinny", "gemm_library", "gemm_tiles"] if dtype == torch.bfloat16 else []))
        self.rowwise = library("rowwise")
        self.rope = library("rope_cache")
        self.attn_generic = library("attention_generic")
        self.gemm_plain = library("gemm_plain")
        self.sampling = library("sampling")
        self.gemm_skinny = library("gemm_skinny") if dtype == torch.bfloat16 else None
        self.gemm_library = None
        self.few_rows = _FEW_ROWS
        self.library_widths = library_widths()
        self._warned_widths = set()
        # compute units of this device: what the attention planner spreads waves over
        self.units = int(torch.cuda.get_device_properties(self.device).multi_processor_count) or _CHIP_UNITS
        if dtype == torch.bfloat16:
            self.gemm_skinny.cdll.tis_gemm_skinny_units(self.units)
            self.gemm_tiles = library("gemm_tiles")
            self.gemm_tiles.cdll.tis_gemm_tiles_units(self.units)
            self.gemm_library = library("gemm_library")
            with torch.cuda.device(self.device):
                self.gemm_library.tis_gemm_library_init()
        self._attn_mfma = {}               # head size -> library
        # partial results of split key ranges: one buffer of fixed size that never moves (captured graphs hold its address)
        self._workspace = torch.empty(_ATTN_WORKSPACE_FLOATS, dtype=torch.float32, device=self.device) \
            if dtype == torch.bfloat16 else None

    # ---- planning on the host --------------------------------------------------------------------------
    def plan_attention_mode(self, seq_rows, window: int = 0):
        """What kind of plan a step gets, from its first stage's rows: two steps may share a captured graph only if
        this is equal. "uneven": single rows of requests that differ widely in length (in what a row sees of its
        request, where the mixer has a window)."""
        return "uneven" if self.dtype == torch.bfloat16 and uneven_lengths(seq_rows, window) else None

    def plan_attention(self, n_heads: int, n_kv_heads: int, head_dim: int, seq_rows, add, mode=None, window: int = 0):
        """An attention mixer's host planning, called while a step's arrays are packed: the work items of the
        matrix-core kernels for the step's rows. Returns {name: (packed array id, host values...)}."""
        plans = {}
        if self.dtype == torch.bfloat16:
            group, cols = n_heads // n_kv_heads, tile_columns(head_dim)
            if (mode == "uneven" and group <= 64 and planned_list_pays(len(seq_rows), n_kv_heads)
                    and all(n == 1 for _, _, n in seq_rows)):
                entries, most = decode_items(seq_rows, n_heads, n_kv_heads, head_dim, window=window, units=self.units)
                return {("attention_decode_items", group, cols, n_kv_heads, window): (add(entries), len(entries), most)}
            nb, items, tiles, steps = attention_items(seq_rows, group, cols, n_kv_heads)
            beside = planned_beside_tiles(seq_rows, items, tiles, steps, n_heads, n_kv_heads, head_dim, window, self.units)
            if beside is not None:
                # one array: the planned entries of four integers, then the tiles' lines of two
                entries, most = beside
                plans[("attention_items", group, cols, n_kv_heads, window)] = (
                    add(np.concatenate((entries.reshape(-1), tiles.reshape(-1)))), len(entries), 1, len(tiles), steps, most)
            elif nb <= 4 and (len(items) or len(tiles)):
                # one array: the items' lines, then the tiles'
                # (a mixer with a window plans for itself: its lists are the same, its keys are its own)
                plans[("attention_items", group, cols, n_kv_heads, window)] = (add(np.concatenate((items, tiles))), len(items),
                                                                       nb, len(tiles), steps, 0)
        return plans

    # ---- helpers -------------------------------------------------------------------------------------
    def _stream(self):
        # torch's current stream of the device (under a graph capture: the capturing stream), by the short way:
        # a kernel launch asks for it, and the public accessor builds a stream object each time (4 us)
        return c_void_p(torch._C._cuda_getCurrentRawStream(self._device_index))

    def _check(self, t: torch.Tensor, what: str, dtype=None):
        dtype = dtype or self.dtype
        if t.device != self.device and not (t.device.type == self.device.type and
                                            (t.device.index or 0) == (self.device.index or 0)):
            raise KernelError(f"{what}: tensor is on {t.device}, engine on {self.device}")
        if t.dtype != dtype:
            raise KernelError(f"{what}: dtype {t.dtype}, expected {dtype}")
        return t

    def _index(self, t: torch.Tensor, what: str, n: Optional[int] = None):
        self._check(t, what, torch.int32)
        if not t.is_contiguous():
            raise KernelError(f"{what}: index tensor must be contiguous")
        if n is not None and t.numel() < n:
            raise KernelError(f"{what}: {t.numel()} entries for {n} rows")
        return t

    def empty(self, *shape, dtype=None):
        """An uninitialised tensor. Rows of bfloat16 activations that may go into the library's product are allocated
        up to the row count the library is asked for (library_rows), so that the product can run on them as they
        lie; the tensor that comes back shows the rows asked for."""
        dtype = dtype or self.dtype
        if len(shape) == 2 and dtype == torch.bfloat16 and shape[0] > self.few_rows:
            rows = library_rows(shape[0])
            if rows != shape[0]:
                return torch.empty(rows, shape[1], dtype=dtype, device=self.device)[:shape[0]]
        return torch.empty(*shape, dtype=dtype, device=self.device)

    # ---- row-wise ------------------------------------------------------------------------------------
    def embedding(self, table, tokens, out=None):
        self._check(table, "embedding table")
        n = tokens.numel()
        self._index(tokens, "tokens")
        D = table.shape[1]
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "embedding out"), "embedding out")
        if out.shape[0] < n or out.shape[1] != D or not table.is_contiguous():
            raise KernelError(f"embedding: out {tuple(out.shape)} does not fit {n} rows of {D}")
        self.rowwise.tis_embedding(self.code, _ptr(table), _ptr(tokens), _ptr(out), out.stride(0), n, D,
                                   self._stream())
        return out

    def rmsnorm(self, x, gain, eps: float, out=None):
        _rows_view(self._check(x, "rmsnorm x"), "rmsnorm x")
        self._check(gain, "rmsnorm gain", torch.float32)
        n, D = x.shape
        if gain.numel() != D or not gain.is_contiguous():
            raise KernelError(f"rmsnorm: gain has {gain.numel()} entries for width {D}")
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "rmsnorm out"), "rmsnorm out")
        if tuple(out.shape) != (n, D):
            raise KernelError(f"rmsnorm: out {tuple(out.shape)} vs x {tuple(x.shape)}")
        self.rowwise.tis_rmsnorm(self.code, _ptr(x), x.stride(0), _ptr(gain), _ptr(out), out.stride(0), n, D,
                                 float(eps), self._stream())
        return out

    def embedding_rmsnorm(self, table, tokens, gain, eps: float, out=None):
        self._check(table, "embedding table")
        self._check(gain, "rmsnorm gain", torch.float32)
        self._index(tokens, "tokens")
        n, D = tokens.numel(), table.shape[1]
        if gain.numel() != D or not gain.is_contiguous() or not table.is_contiguous():
            raise KernelError(f"embedding_rmsnorm: gain has {gain.numel()} entries for width {D}")
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "embedding_rmsnorm out"), "embedding_rmsnorm out")
        if out.shape[0] < n or out.shape[1] != D:
            raise KernelError(f"embedding_rmsnorm: out {tuple(out.shape)} does not fit {n} rows of {D}")
        self.rowwise.tis_embedding_rmsnorm(self.code, _ptr(table), _ptr(tokens), _ptr(gain), _ptr(out),
                                           out.stride(0), n, D, float(eps), self._stream())
        return out

    def gather_rows(self, src, state, index, out=None):
        """out[r] = src[index[r]] if index[r] >= 0 else state[-index[r]-1]."""
        _rows_view(self._check(src, "gather src"), "gather src")
        _rows_view(self._check(state, "gather state"), "gather state")
        n = index.numel()
        self._index(index, "gather index")
        D = src.shape[1]
        if state.shape[1] != D:
            raise KernelError(f"gather_rows: src width {D}, state width {state.shape[1]}")
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "gather out"), "gather out")
        if out.shape[0] < n or out.shape[1] != D:
            raise KernelError(f"gather_rows: out {tuple(out.shape)} does not fit {n} rows of {D}")
        self.rowwise.tis_gather_rows(self.code, _ptr(src), src.stride(0), _ptr(state), state.stride(0), _ptr(index),
                                     _ptr(out), out.stride(0), n, D, self._stream())
        return out

    def copy_rows(self, src, src_index, dst, dst_index):
        """dst[dst_index[i]] = src[src_index[i]]."""
        _rows_view(self._check(src, "copy src"), "copy src")
        _rows_view(self._check(dst, "copy dst"), "copy dst")
        n = src_index.numel()
        self._index(src_index, "copy src_index")
        self._index(dst_index, "copy dst_index", n)
        if src.shape[1] != dst.shape[1]:
            raise KernelError(f"copy_rows: widths {src.shape[1]} and {dst.shape[1]}")
        self.rowwise.tis_copy_rows(self.code, _ptr(src), src.stride(0), _ptr(src_index), _ptr(dst), dst.stride(0),
                                   _ptr(dst_index), n, src.shape[1], self._stream())

    def swiglu(self, gu, out=None):
        """out[:, f] = silu(gu[:, 2f]) * gu[:, 2f + 1]: gate and up columns interleaved."""
        _rows_view(self._check(gu, "swiglu in"), "swiglu in")
        n, F2 = gu.shape
        if F2 % 2:
            raise KernelError(f"swiglu: input width {F2} is odd")
        F = F2 // 2
        if out is None:
            out = self.empty(n, F)
        _rows_view(self._check(out, "swiglu out"), "swiglu out")
        if tuple(out.shape) != (n, F):
            raise KernelError(f"swiglu: out {tuple(out.shape)} for {n} rows of {F}")
        self.rowwise.tis_swiglu(self.code, _ptr(gu), gu.stride(0), _ptr(out), out.stride(0), n, F, self._stream())
        return out

    # ---- matrix products -----------------------------------------------------------------------------
    def linear(self, x, w, residual=None, out_dtype=None, rms=None, reuse_residual=False):
        """f(x)[M,K] . w[N,K]^T (+ residual[M,N]); `out_dtype` float32 gives 32-bit results from bfloat16 inputs.

        rms = (gain, eps): f is the RMSNorm of the rows, fused into the product where the kernel allows.
        reuse_residual: the caller has no further use for `residual`; an operations object may then write the result
        over it. This one never does: every product's result has memory of its own.
        """
        _rows_view(self._check(x, "linear x"), "linear x")
        self._check(w, "linear w")
        out_dtype = out_dtype or self.dtype
        M, K = x.shape
        if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
            raise KernelError(f"linear: x {tuple(x.shape)} against w {tuple(w.shape)} (w is [out, in], contiguous)")
        N = w.shape[0]
        if residual is not None:
            _rows_view(self._check(residual, "linear residual", out_dtype), "linear residual")
            if tuple(residual.shape) != (M, N):
                raise KernelError(f"linear: residual {tuple(residual.shape)} for result {(M, N)}")
        if rms is not None:
            self._check(rms[0], "rmsnorm gain", torch.float32)
            if rms[0].numel() != K or not rms[0].is_contiguous():
                raise KernelError(f"linear: norm gain has {rms[0].numel()} entries for width {K}")
        if self.dtype == torch.float32:
            if rms is not None:
                x = self.rmsnorm(x, rms[0], rms[1])
            out = self.empty(M, N, dtype=torch.float32)
            self.gemm_plain.tis_gemm_plain(0, 0, _ptr(x), x.stride(0), _ptr(w), K, _ptr(residual),
                                           residual.stride(0) if residual is not None else 0, _ptr(out), N, M, N, K,
                                           self._stream())
            return out
        route = self._route(x, M, N, K, out_dtype, residual)
        if route == "few_rows":
            out = self.empty(M, N, dtype=out_dtype)
            if out_dtype == torch.float32 and residual is not None:
                raise KernelError("linear: a 32-bit result of bfloat16 operands takes no residual")
            self.gemm_skinny.tis_gemm_skinny(
                _ptr(x), x.stride(0), _ptr(w), _ptr(rms[0] if rms else None), float(rms[1]) if rms else 0.0,
                _ptr(residual), residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0), M, N, K,
                1 if residual is not None else 0, _DT[out_dtype], self._stream())
            return out
        if rms is not None:
            x = self.rmsnorm(x, rms[0], rms[1])
        if route == "library":
            return self._linear_library(x, w, residual)
        if route == "tiles":
            if out_dtype == torch.float32 and residual is not None:
                raise KernelError("linear: a 32-bit result of bfloat16 operands takes no residual")
            out = self.empty(M, N, dtype=out_dtype)
            self.gemm_tiles.tis_gemm_tiles(_ptr(x), x.stride(0), _ptr(w), _ptr(residual),
                                           residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0),
                                           M, N, K, 1 if out_dtype == torch.float32 else 0, self._stream())
            return out
        out = self.empty(M, N, dtype=out_dtype)
        self.gemm_plain.tis_gemm_plain(1, _DT[out_dtype], _ptr(x), x.stride(0), _ptr(w), K, _ptr(residual),
                                       residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0), M, N,
                                       K, self._stream())
        return out

    def _route(self, x, M, N, K, out_dtype=None, residual=None):
        """Which kernel takes this bfloat16 product (see product_route); says once per width that a product of many
        rows runs on the few-row kernel because the library's list does not hold its widths."""
        aligned = K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
        route = product_route(M, N, K, aligned, out_dtype == torch.float32, self.library_widths, self.few_rows)
        if route == "library" and residual is not None and (residual.stride(0) % 8 or residual.data_ptr() % 16):
            route = "few_rows"
        if route == "tiles" and residual is not None and (residual.stride(0) % 4 or residual.data_ptr() % 8):
            route = "few_rows"
        if route == "few_rows" and M > 8 * self.few_rows and (N, K) not in self._warned_widths \
                and out_dtype != torch.float32:
            self._warned_widths.add((N, K))
            print(f"[tis-amd] a product of {M} rows with {N} output and {K} input columns runs on the few-row kernel: "
                  f"these widths are not in {os.path.basename(_WIDTHS_FILE)} (the widths the library's product has "
                  f"been tested at)", file=__import__("sys").stderr, flush=True)
        return route

    def _few_rows_ok(self, x, M, N, K):
        return self.dtype == torch.bfloat16 and M > 0 and self._route(x, M, N, K) == "few_rows"

    def linear_swiglu(self, x, w, rms=None):
        """silu(g) * u of the rows of f(x) . w^T, w holding gate and up rows interleaved: [M, N/2]."""
        _rows_view(self._check(x, "linear x"), "linear x")
        M, K = x.shape
        if w.dim() == 2 and w.shape[0] % 2 == 0 and self._few_rows_ok(x, M, w.shape[0], K):
            self._check(w, "linear w")
            if w.shape[1] != K or not w.is_contiguous():
                raise KernelError(f"linear: x {tuple(x.shape)} against w {tuple(w.shape)} (w is [out, in], contiguous)")
            if rms is not None and (rms[0].numel() != K or rms[0].dtype != torch.float32):
                raise KernelError(f"linear: norm gain has {rms[0].numel()} entries for width {K}")
            N = w.shape[0]
            out = self.empty(M, N // 2)
            self.gemm_skinny.tis_gemm_skinny(
                _ptr(x), x.stride(0), _ptr(w), _ptr(rms[0] if rms else None), float(rms[1]) if rms else 0.0,
                _ptr(None), 0, _ptr(out), out.stride(0), M, N, K, 2, 1, self._stream())
            return out
        return self.swiglu(self.linear(x, w, rms=rms))

    @staticmethod
    def _holds_rows(t, rows: int) -> bool:
        """Whether `rows` rows of t's stride lie inside the memory behind t."""
        last = t.storage_offset() + (rows - 1) * t.stride(0) + t.shape[1]
        return last * t.element_size() <= t.untyped_storage().nbytes()

    def _with_rows(self, t, rows: int):
        """t itself if the memory behind it holds `rows` rows (tensors from `empty` do), else a copy that does."""
        if self._holds_rows(t, rows):
            return t
        c = self.empty(t.shape[0], t.shape[1], dtype=t.dtype)
        c.copy_(t)
        return c

    def _linear_library(self, x, w, residual):
        """The library's product for many rows (reference main_models_new.py:19-20 uses one too), asked at
        library_rows(M) rows: the operands' memory reaches that far, and the rows beyond M are not looked at again.
        The result has memory of its own, also where the caller has no further use for the residual."""
        M, K = x.shape
        N = w.shape[0]
        rows = library_rows(M)
        if (N, K) not in self.library_widths:
            raise KernelError(f"linear: widths ({N}, {K}) are not among those the library's product is used at")
        x = self._with_rows(x, rows)
        if residual is not None:
            residual = self._with_rows(residual, rows)
        out = self.empty(M, N)
        if not self._holds_rows(out, rows):
            raise KernelError(f"linear: the result of {M} rows has no room for {rows}")
        self.gemm_library.tis_gemm_library(_ptr(x), x.stride(0), _ptr(w), _ptr(residual),
                                           residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0),
                                           rows, N, K, 0, self._stream())
        return out

    # ---- position encoding + cache write, attention --------------------------------------------------
    def rope_write_kv(self, qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                      interleaved=False, write_cache=True, paired=False, q_out=None):
        """Rotate q (in place, or into `q_out`) and write rotated k and v into the cache plane.

        paired: the q and k heads of `qkv` hold the members of each rotary pair side by side (pair j at columns
        2j, 2j+1), as a projection with pair-ordered weight rows leaves them; `q_out` then receives the queries
        in natural order.
        """
        _rows_view(self._check(qkv, "qkv"), "qkv")
        if paired and q_out is None:
            raise KernelError("rope_write_kv: paired input needs q_out")
        if q_out is not None:
            _rows_view(self._check(q_out, "q_out"), "q_out")
            if tuple(q_out.shape) != (qkv.shape[0], n_heads * head_dim):
                raise KernelError(f"rope_write_kv: q_out {tuple(q_out.shape)} for {qkv.shape[0]} rows of {n_heads * head_dim}")
        n = qkv.shape[0]
        if qkv.shape[1] != (n_heads + 2 * n_kv_heads) * head_dim:
            raise KernelError(f"rope_write_kv: row width {qkv.shape[1]} is not (heads {n_heads} + 2 x kv heads "
                              f"{n_kv_heads}) x head size {head_dim}")
        self._index(positions, "positions", n)
        if table is not None:
            self._check(table, "rotary table", torch.float32)
            if table.dim() != 3 or table.shape[1] != head_dim // 2 or table.shape[2] != 2 or not table.is_contiguous():
                raise KernelError(f"rope_write_kv: table {tuple(table.shape)} for head size {head_dim}")
        if write_cache:
            self._index(write_slots, "write_slots", n)
            self._check_plane(plane, n_kv_heads, head_dim, page_size)
        self.rope.tis_rope_write_kv(self.code, _ptr(qkv), qkv.stride(0), _ptr(positions),
                                    _ptr(write_slots if write_cache else None), _ptr(table),
                                    _ptr(plane if write_cache else None), n, n_heads, n_kv_heads, head_dim, page_size,
                                    int(bool(interleaved)), int(bool(write_cache)), int(bool(paired)), _ptr(q_out),
                                    q_out.stride(0) if q_out is not None else 0, self._stream())

    def qkv_rope(self, x, w, rms, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                 interleaved=False, write_cache=True):
        """Queries [rows, heads*head_dim], rotated, of f(x) . w^T; rotated keys and values go into the cache plane.

        w: [(heads + 2 kv heads) * head_dim, K] with the rows of every q and k head in pair order. For few rows in
        bfloat16 this is one kernel; otherwise the projection followed by the rotary/cache-write kernel.
        """
        _rows_view(self._check(x, "qkv x"), "qkv x")
        self._check(w, "qkv w")
        M, K = x.shape
        N = (n_heads + 2 * n_kv_heads) * head_dim
        if w.dim() != 2 or tuple(w.shape) != (N, K) or not w.is_contiguous():
            raise KernelError(f"qkv_rope: w {tuple(w.shape)} is not [{N}, {K}] contiguous")
        if self._few_rows_ok(x, M, N, K) and head_dim % 4 == 0:
            self._index(positions, "positions", M)
            if table is not None:
                self._check(table, "rotary table", torch.float32)
                if table.dim() != 3 or table.shape[1] != head_dim // 2 or table.shape[2] != 2 or not table.is_contiguous():
                    raise KernelError(f"qkv_rope: table {tuple(table.shape)} for head size {head_dim}")
            if write_cache:
                self._index(write_slots, "write_slots", M)
                self._check_plane(plane, n_kv_heads, head_dim, page_size)
            if rms is not None and (rms[0].numel() != K or rms[0].dtype != torch.float32):
                raise KernelError(f"qkv_rope: norm gain has {rms[0].numel()} entries for width {K}")
            q = self.empty(M, n_heads * head_dim)
            self.gemm_skinny.tis_gemm_skinny_qkv_rope(
                _ptr(x), x.stride(0), _ptr(w), _ptr(rms[0] if rms else None), float(rms[1]) if rms else 0.0, _ptr(q),
                q.stride(0), M, K, _ptr(positions), _ptr(write_slots if write_cache else None), _ptr(table),
                _ptr(plane if write_cache else None), n_heads, n_kv_heads, head_dim, page_size,
                int(bool(interleaved)), int(bool(write_cache)), self._stream())
            return q
        qkv = self.linear(x, w, rms=rms)
        q = self.empty(M, n_heads * head_dim)
        self.rope_write_kv(qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                           interleaved, write_cache, paired=True, q_out=q)
        return q

    def _check_plane(self, plane, n_kv_heads, head_dim, page_size):
        self._check(plane, "cache plane")
        if plane.dim() != 5 or tuple(plane.shape[1:]) != (2, n_kv_heads, page_size, head_dim) or \
                not plane.is_contiguous():
            raise KernelError(f"cache plane {tuple(plane.shape)} is not [pages, 2, {n_kv_heads}, {page_size}, "
                              f"{head_dim}] contiguous")

    def paged_attention(self, q, plane, batch, group, n_heads, n_kv_heads, head_dim, window=0, scale=None,
                        slopes=None, sink=False, gate=None):
        """Attention of the rows in `batch` over the cache plane; `q` is [rows, heads*head_dim] (a strided view is fine).

        `batch` brings positions, row_seq and the group's block tables; `group` names the page group. `slopes`
        ([heads] 32-bit, or None): a bias slope[h] * (key position - row position) on the scores; such calls go to
        the general kernel. sink: the softmax's denominator also counts a key of score 0 that has no value. gate
        ([rows, heads] 32-bit, a strided view is fine): head h's result is multiplied by sigmoid(gate[:, h]). Calls with
        a sink or a gate that the matrix-core kernels do not take go to the kernel for keys and values of any sizes.
        window > 0: a row sees its last `window` keys; window < 0: the keys of its own chunk of -window positions, the
        chunks' edges at multiples of that size in the request (such calls, too, go to the kernel for any sizes where the matrix-core kernels do not
        take them); 0: all.
        """
        group_name = group
        if (sink or gate is not None) and slopes is not None:
            raise KernelError("attention: score slopes go with neither a sink nor a gate")
        _rows_view(self._check(q, "q"), "q")
        n = q.shape[0]
        page_size = plane.shape[3]
        self._check_plane(plane, n_kv_heads, head_dim, page_size)
        if q.shape[1] != n_heads * head_dim:
            raise KernelError(f"attention: q width {q.shape[1]} is not heads {n_heads} x head size {head_dim}")
        tables = batch.block_tables[group]
        self._check(tables, "block tables", torch.int32)
        if tables.dim() != 2 or tables.stride(1) != 1:
            raise KernelError(f"attention: block tables {tuple(tables.shape)} must be 2-d")
        self._index(batch.positions, "positions", n)
        self._index(batch.row_seq, "row_seq", n)
        if batch.max_kv_len > tables.shape[1] * page_size:
            raise KernelError(f"attention: a row sees {batch.max_kv_len} keys but block tables cover "
                              f"{tables.shape[1] * page_size}")
        if scale is None:
            scale = head_dim ** -0.5
        out = self.empty(n, n_heads * head_dim)
        if n == 0:
            return out
        group = n_heads // n_kv_heads
        if slopes is not None:
            self._check(slopes, "score slopes", torch.float32)
            if slopes.numel() != n_heads or not slopes.is_contiguous():
                raise KernelError(f"attention: {slopes.numel()} score slopes for {n_heads} heads")
        if (slopes is None and self.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256 and page_size % 16 == 0
                and group <= 64 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0):
            cols = tile_columns(head_dim)
            planned = batch.extras.get(("attention_decode_items", group, cols, n_kv_heads, int(window)))
            plan = batch.extras.get(("attention_items", group, cols, n_kv_heads, int(window)))
            if planned is None and plan is None:
                # a caller that did not plan (a kernel test): plan now, tiles wherever they fit
                if uneven_lengths(batch.seq_rows, int(window)) and planned_list_pays(n, n_kv_heads):
                    entries, most = decode_items(batch.seq_rows, n_heads, n_kv_heads, head_dim, window=int(window),
                                                 units=self.units)
                    planned = (torch.from_numpy(entries).reshape(-1).to(self.device), len(entries), most)
                else:
                    nb, host_items, host_tiles, steps = attention_items(batch.seq_rows, group, cols)
                    beside = planned_beside_tiles(batch.seq_rows, host_items, host_tiles, steps, n_heads, n_kv_heads,
                                                  head_dim, int(window), self.units)
                    if beside is not None:
                        both = np.concatenate((beside[0].reshape(-1), host_tiles.reshape(-1)))
                        plan = (torch.from_numpy(np.ascontiguousarray(both)).to(self.device), len(beside[0]), 1,
                                len(host_tiles), steps, beside[1])
                    else:
                        both = np.ascontiguousarray(np.concatenate((host_items, host_tiles)))
                        plan = (torch.from_numpy(both).reshape(-1).to(self.device), len(host_items), nb, len(host_tiles),
                                steps, 0)
            planned_splits = 0
            if planned is not None:
                # single rows with splits planned row by row: one entry of four integers per wave
                lines, n_items, planned_splits = planned
                lines = lines.reshape(-1)
                if batch.max_seq_rows > 1 or lines.numel() != 4 * n_items:
                    raise KernelError(f"attention: a planned list of {lines.numel()} integers for {n_items} entries "
                                      f"of single rows ({batch.max_seq_rows} rows a request)")
                items, tiles, n_tiles, tile_steps, nb = lines, None, 0, (0, 0), 1
                while group > 16 * nb:
                    nb *= 2
            else:
                lines, n_items, nb, n_tiles, tile_steps, planned_splits = plan
                lines = lines.reshape(-1)
                width = 4 if planned_splits else 2      # a planned entry, or an item's (first row, rows)
                if lines.numel() < width * n_items + 2 * n_tiles:
                    raise KernelError(f"attention: the work list holds {lines.numel()} integers for {n_items} items "
                                      f"and {n_tiles} tiles")
                items = lines[:width * n_items] if n_items else None
                tiles = lines[width * n_items:] if n_tiles else None
                if planned_splits:
                    while group > 16 * nb:
                        nb *= 2
                elif batch.max_seq_rows <= 1 and n_items == n:
                    items = None        # single rows in order: the kernel needs no list
            lib = self._attn_mfma.get(head_dim)
            if lib is None:
                lib = self._attn_mfma[head_dim] = library(f"attention_mfma@{head_dim}")
                with torch.cuda.device(self.device):
                    lib.tis_attention_mfma_side_stream(c_void_p(_side_stream(self._device_index).cuda_stream))
                built = lib.cdll.tis_attention_mfma_tile_columns()
                if built != cols:
                    raise KernelError(f"attention: the kernel's tiles hold {built} columns a wave, the planner "
                                      f"assumes {cols}")
            single = items is None and n_tiles == 0
            lp = attention_launch_plan(n, n_items, n_tiles, tile_steps, single, batch.max_kv_len, n_heads, n_kv_heads,
                                       head_dim, planned_splits=planned_splits, units=self.units)
            n_splits, min_steps, tile_splits, tile_max_steps = lp.n_splits, lp.min_steps, lp.tile_splits, lp.tile_max_steps
            part_o = part_ml = row_splits = None
            if lp.stride > 1:
                if lp.need_floats > self._workspace.numel():
                    raise KernelError(f"attention: {lp.need_floats} floats of partial results for a workspace of "
                                      f"{self._workspace.numel()}")
                part_o = self._workspace
                part_ml = self._workspace[lp.ml_offset:]
                if lp.min_steps != 0 or n_tiles:
                    row_splits = self._workspace[lp.row_splits_offset:]
            if lines.dtype != torch.int32 or not lines.is_contiguous():
                raise KernelError("attention: the work list must be contiguous 32-bit integers")
            lib.tis_attention_mfma_sink(_ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0),
                                        _ptr(batch.row_seq), _ptr(batch.positions), _ptr(items), n_items, nb, _ptr(tiles),
                                        n_tiles, _ptr(out), out.stride(0), _ptr(part_o), _ptr(part_ml), n, n_heads,
                                        n_kv_heads, head_dim, page_size, int(window), float(scale), n_splits, min_steps,
                                        tile_splits, tile_max_steps, _ptr(row_splits), 1 if sink else 0, self._stream())
            if gate is not None:
                self.head_gate(out, gate, n_heads, head_dim)
            return out
        if sink or gate is not None or window < 0:
            if slopes is not None:
                raise KernelError("attention: score slopes do not go with chunks of positions")
            return self.paged_attention_kv(q, plane, batch, group_name, n_heads, n_kv_heads, head_dim, head_dim, page_size,
                                           max(0, window), scale, sink=sink, gate=gate, chunk=max(0, -window))
        self.attn_generic.tis_attention_generic(
            self.code, _ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0), _ptr(batch.row_seq),
            _ptr(batch.positions), _ptr(out), out.stride(0), n, n_heads, n_kv_heads, head_dim, page_size, int(window),
            float(scale), _ptr(slopes), self._stream())
        return out

    # ---- a residual stream in 32-bit, norm after the sum ------------------------------------------------
    # The libraries below are loaded when a model first asks for them: a model that has no such part never
    # compiles them.
    def _lazy(self, name):
        lib = self.__dict__.get("_lib_" + name)
        if lib is None:
            lib = self.__dict__["_lib_" + name] = library(name)
        return lib

    def _f32(self, t, what, n=None):
        self._check(t, what, torch.float32)
        if not t.is_contiguous() or (n is not None and t.numel() != n):
            raise KernelError(f"{what}: expected {n if n is not None else 'some'} contiguous 32-bit floats, got "
                              f"{tuple(t.shape)}")
        return t

    def _f32_rows(self, t, what, rows, cols):
        _rows_view(self._check(t, what, torch.float32), what)
        if t.shape[0] != rows or t.shape[1] < cols:
            raise KernelError(f"{what}: {tuple(t.shape)} for {rows} rows of at least {cols}")
        return t

    def embed_scaled(self, table, tokens, scale: float):
        """(x32, x): rows of the table times `scale` in 32-bit, and the same rows in the compute type (in a 32-bit
        engine both are one tensor)."""
        self._check(table, "embedding table")
        self._index(tokens, "tokens")
        n, D = tokens.numel(), table.shape[1]
        if not table.is_contiguous():
            raise KernelError("embed_scaled: the table must be contiguous")
        x32 = torch.empty(n, D, dtype=torch.float32, device=self.device)
        x = x32 if self.dtype == torch.float32 else self.empty(n, D)
        self._lazy("stream32").tis_embed_scale(self.code, _ptr(table), _ptr(tokens), float(scale), _ptr(x32),
                                               _ptr(None if x is x32 else x), n, D, self._stream())
        return x32, x

    def gated_postnorm(self, x32, branches, gate, gate_bias, alpha: float, gain, eps: float):
        """norm(alpha * x32 + sigmoid(gate + gate_bias) * sum_i scale_i * y_i) with an RMS norm (eps under the root):
        (result in 32-bit, result in the compute type). branches: one or two (y [rows, width] 32-bit, scale);
        gate: [rows, width] 32-bit (a strided view is fine) or None for no gate."""
        n, D = x32.shape
        self._f32(x32, "gated_postnorm x", n * D)
        if not 1 <= len(branches) <= 2:
            raise KernelError(f"gated_postnorm: {len(branches)} branches (one or two)")
        for y, _ in branches:
            self._f32_rows(y, "gated_postnorm branch", n, D)
        if gate is not None:
            self._f32_rows(gate, "gated_postnorm gate", n, D)
            if gate_bias is not None:
                self._f32(gate_bias, "gated_postnorm gate bias", D)
        self._f32(gain, "gated_postnorm gain", D)
        out32 = torch.empty(n, D, dtype=torch.float32, device=self.device)
        out = out32 if self.dtype == torch.float32 else self.empty(n, D)
        (y0, s0), (y1, s1) = branches[0], (branches[1] if len(branches) > 1 else (None, 0.0))
        self._lazy("stream32").tis_gated_postnorm(
            self.code, _ptr(x32), _ptr(y0), y0.stride(0), float(s0), _ptr(y1), y1.stride(0) if y1 is not None else 0,
            float(s1), _ptr(gate), gate.stride(0) if gate is not None else 0, _ptr(gate_bias if gate is not None else None),
            float(alpha), _ptr(gain), float(eps), _ptr(out32), _ptr(None if out is out32 else out), n, D, self._stream())
        return out32, out

    def rmsnorm32(self, x32, gain, eps: float):
        """x / sqrt(mean(x^2) + eps) * gain of 32-bit rows, in the compute type."""
        n, D = x32.shape
        self._f32(x32, "rmsnorm32 x", n * D)
        self._f32(gain, "rmsnorm32 gain", D)
        out = self.empty(n, D)
        self._lazy("stream32").tis_rmsnorm32(self.code, _ptr(x32), _ptr(gain), float(eps), _ptr(out), out.stride(0), n, D,
                                             self._stream())
        return out

    def head_norm_gate(self, o32, gate, gain, n_heads: int, vdim: int, eps: float, act: str):
        """Per head: o / sqrt(mean(o^2) + eps) * gain * act(gate), in the compute type. o32, gate: [rows, heads*vdim]
        32-bit (gate may be a strided view); gain: [vdim] shared by the heads or [heads*vdim]; act: "silu" or
        "sigmoid"."""
        n = o32.shape[0]
        W = n_heads * vdim
        self._f32_rows(o32, "head_norm_gate o", n, W)
        self._f32_rows(gate, "head_norm_gate gate", n, W)
        self._check(gain, "head_norm_gate gain", torch.float32)
        if gain.numel() not in (vdim, W) or not gain.is_contiguous() or act not in ("silu", "sigmoid"):
            raise KernelError(f"head_norm_gate: gain of {gain.numel()} for {n_heads} heads of {vdim}, act {act!r}")
        out = self.empty(n, W)
        self._lazy("stream32").tis_head_norm_gate(
            self.code, _ptr(o32), o32.stride(0), _ptr(gate), gate.stride(0), _ptr(gain),
            int(gain.numel() == W and n_heads > 1), 0 if act == "silu" else 1, float(eps), _ptr(out), out.stride(0), n,
            n_heads, vdim, self._stream())
        return out

    def lowrank_decay(self, low, w2, bias, tau: float):
        """sigmoid(low . w2^T + bias)^(1/tau) in 32-bit: low [rows, rank] (a strided view is fine), w2 [channels, rank]."""
        n, rank = low.shape
        _rows_view(self._check(low, "lowrank_decay low", torch.float32), "lowrank_decay low")
        C = w2.shape[0]
        self._f32(w2, "lowrank_decay w2", C * rank)
        self._f32(bias, "lowrank_decay bias", C)
        out = torch.empty(n, C, dtype=torch.float32, device=self.device)
        self._lazy("stream32").tis_lowrank_decay(_ptr(low), low.stride(0), rank, _ptr(w2), _ptr(bias), float(tau),
                                                 _ptr(out), n, C, self._stream())
        return out

    def layernorm32(self, x32, gain, bias, eps: float):
        """(x - mean) / sqrt(var + eps) * gain + bias of 32-bit rows, in the compute type (bias may be None)."""
        n, D = x32.shape
        self._f32(x32, "layernorm32 x", n * D)
        self._f32(gain, "layernorm32 gain", D)
        if bias is not None:
            self._f32(bias, "layernorm32 bias", D)
        out = self.empty(n, D)
        self._lazy("stream32").tis_layernorm32(self.code, _ptr(x32), _ptr(gain), _ptr(bias), float(eps), _ptr(out),
                                               out.stride(0), n, D, self._stream())
        return out

    def residual_norm(self, x32, y=None, y_rms=None, copy=False, norm=None):
        """x32 <- x32 + y, in place, with what usually follows: (x32, copy, normed).

        y may also be a `ChosenExperts` (what routed_experts gives with combine=False): the weighted sum of a row's
        chosen experts is then taken inside this kernel.

        y: [rows, width] 32-bit (a strided view is fine) or None; y_rms = (gain, eps): y is RMS-normed with that gain
        before it is added. copy: also return the new rows in the compute type. norm = (kind, gain, bias, eps) with kind
        "layer" (bias may be None) or "rms": also return the norm of the new rows in the compute type. In a 32-bit
        engine the copy is the stream itself."""
        n, D = x32.shape
        self._f32(x32, "residual_norm x", n * D)
        chosen = None
        if isinstance(y, ChosenExperts):
            chosen, y = y, y.results
            top = chosen.ids.shape[1]
            self._index(chosen.ids, "expert ids", n * top)
            self._f32(chosen.weights, "expert weights", n * top)
            _rows_view(self._check(chosen.rows, "experts' input rows"), "experts' input rows")
            if tuple(chosen.rows.shape) != (n, D) or (y is not None and tuple(y.shape) != (n * top, D)):
                raise KernelError(f"residual_norm: experts' results {None if y is None else tuple(y.shape)} and rows "
                                  f"{tuple(chosen.rows.shape)} for {n} rows of {D} with {top} choices")
            if y is not None:
                self._f32_rows(y, "experts' results", n * top, D)
            if chosen.extra is not None:
                self._f32_rows(chosen.extra, "what every row adds beside its choices", n, D)
                self._f32_rows(chosen.extra_gate, "that term's gate", n, 1)
        elif y is not None:
            self._f32_rows(y, "residual_norm y", n, D)
        elif y_rms is not None:
            raise KernelError("residual_norm: a norm on a branch that is not there")
        if y_rms is not None:
            self._f32(y_rms[0], "residual_norm branch gain", D)
        kind, gain, bias, eps = 0, None, None, 0.0
        if norm is not None:
            kind = {"layer": 1, "rms": 2}[norm[0]]
            gain, bias, eps = norm[1], norm[2], norm[3]
            self._f32(gain, "residual_norm gain", D)
            if bias is not None:
                self._f32(bias, "residual_norm bias", D)
        as_is = self.dtype == torch.float32
        cp = self.empty(n, D) if copy and not as_is else None
        normed = self.empty(n, D) if kind else None
        extra = chosen.extra if chosen is not None else None
        self._lazy("stream32").tis_residual_norm(
            self.code, _ptr(x32), _ptr(y), y.stride(0) if y is not None else 0, _ptr(y_rms[0] if y_rms else None),
            float(y_rms[1]) if y_rms else 0.0, _ptr(x32), _ptr(cp), cp.stride(0) if cp is not None else 0, kind, _ptr(gain),
            _ptr(bias), float(eps), _ptr(normed), normed.stride(0) if normed is not None else 0, n, D,
            _ptr(chosen.ids if chosen else None), _ptr(chosen.weights if chosen else None),
            chosen.ids.shape[1] if chosen else 0, chosen.n_experts if chosen else 0,
            _ptr(chosen.rows if chosen else None), chosen.rows.stride(0) if chosen else 0,
            _ptr(extra), extra.stride(0) if extra is not None else 0, _ptr(chosen.extra_gate if extra is not None else None),
            chosen.extra_gate.stride(0) if extra is not None else 0, self._stream())
        return x32, (x32 if copy and as_is else cp), normed

    _ACTS = {"gelu_tanh": 0, "silu": 1, "sigmoid": 2}

    def gate_table(self, z, table, tokens, act: str):
        """act(z) * table[tokens]: z [rows, W] 32-bit (a strided view is fine), table [entries, W] in the compute type;
        the result [rows, W] in the compute type. act: "gelu_tanh", "silu" or "sigmoid"."""
        n, W = z.shape
        self._f32_rows(z, "gate_table z", n, W)
        _rows_view(self._check(table, "gate_table table"), "gate_table table")
        if table.shape[1] != W:
            raise KernelError(f"gate_table: table rows of {table.shape[1]} for gates of {W}")
        self._index(tokens, "tokens", n)
        out = self.empty(n, W)
        self._lazy("stream32").tis_gate_table(self.code, _ptr(z), z.stride(0), _ptr(table), table.stride(0), _ptr(tokens),
                                              self._ACTS[act], _ptr(out), out.stride(0), n, W, self._stream())
        return out

    def head_gate(self, x, gate, n_heads: int, vdim: int):
        """x[:, h * vdim + (0..vdim)] *= sigmoid(gate[:, h]), in place. x: [rows, heads * vdim] in the compute type;
        gate: [rows, heads] 32-bit (a strided view is fine)."""
        _rows_view(self._check(x, "head_gate x"), "head_gate x")
        n = x.shape[0]
        if x.shape[1] != n_heads * vdim:
            raise KernelError(f"head_gate: x {tuple(x.shape)} for {n_heads} heads of {vdim}")
        self._f32_rows(gate, "head_gate gate", n, n_heads)
        self._lazy("stream32").tis_head_gate(self.code, _ptr(x), x.stride(0), _ptr(gate), gate.stride(0), n, n_heads, vdim,
                                             self._stream())
        return x

    def activate32(self, z, act: str):
        """act on 32-bit rows, in place (z may be a strided view of some columns)."""
        _rows_view(self._check(z, "activate32 z", torch.float32), "activate32 z")
        self._lazy("stream32").tis_activate32(_ptr(z), z.stride(0), self._ACTS[act], z.shape[0], z.shape[1], self._stream())
        return z

    # ---- blocks whose sublayers read one norm of the stream and are summed with a factor per channel --------------
    def dyt32(self, x32, alpha: float, gain, bias=None):
        """Dynamic tanh of 32-bit rows, tanh(alpha * x) * gain + bias element by element, in the compute type."""
        n, D = x32.shape
        self._f32(x32, "dyt32 x", n * D)
        self._f32(gain, "dyt32 gain", D)
        if bias is not None:
            self._f32(bias, "dyt32 bias", D)
        out = self.empty(n, D)
        self._lazy("stream32").tis_dyt32(self.code, _ptr(x32), float(alpha), _ptr(gain), _ptr(bias), _ptr(out), out.stride(0),
                                         n, D, self._stream())
        return out

    def scaled_sum(self, x32, branches, norm=None):
        """x32 <- x32 + sum_i scale_i * (y_i + bias_i), in place: (x32, normed). branches: one or two (y, scale, bias)
        with y [rows, width] 32-bit (a strided view is fine), scale and bias [width] 32-bit or None (1 and 0). The
        second y may be a `ChosenExperts` (a routed feed-forward's results before the sum over a row's choices, which is
        then taken here; weights None: every choice counts once). norm = ("dyt", alpha, gain, bias): also return the
        dynamic tanh of the new rows in the compute type."""
        n, D = x32.shape
        self._f32(x32, "scaled_sum x", n * D)
        if not 1 <= len(branches) <= 2:
            raise KernelError(f"scaled_sum: {len(branches)} branches (one or two)")
        chosen = None
        args = []
        for i, (y, scale, bias) in enumerate(branches):
            if isinstance(y, ChosenExperts):
                if i == 0:
                    raise KernelError("scaled_sum: a routed feed-forward's results come as the second branch")
                chosen, y = y, y.results
                top = chosen.ids.shape[1]
                self._index(chosen.ids, "expert ids", n * top)
                if chosen.weights is not None:
                    self._f32(chosen.weights, "expert weights", n * top)
                _rows_view(self._check(chosen.rows, "experts' input rows"), "experts' input rows")
                if tuple(chosen.rows.shape) != (n, D):
                    raise KernelError(f"scaled_sum: experts' input rows {tuple(chosen.rows.shape)} for {n} rows of {D}")
                if y is not None:
                    self._f32_rows(y, "experts' results", n * top, D)
            else:
                self._f32_rows(y, "scaled_sum branch", n, D)
            for t, what in ((scale, "scaled_sum factors"), (bias, "scaled_sum bias")):
                if t is not None:
                    self._f32(t, what, D)
            args += [_ptr(y), y.stride(0) if y is not None else 0, _ptr(scale), _ptr(bias)]
        if len(branches) == 1:
            args += [_ptr(None), 0, _ptr(None), _ptr(None)]
        kind, alpha, gain, nbias, normed = 0, 0.0, None, None, None
        if norm is not None:
            if norm[0] != "dyt":
                raise KernelError(f"scaled_sum: norm kind {norm[0]!r} (known: 'dyt')")
            kind, alpha, gain, nbias = 3, float(norm[1]), norm[2], norm[3]
            self._f32(gain, "scaled_sum norm gain", D)
            if nbias is not None:
                self._f32(nbias, "scaled_sum norm bias", D)
            normed = self.empty(n, D)
        self._lazy("stream32").tis_scaled_sum(
            self.code, _ptr(x32), *args, _ptr(chosen.ids if chosen else None), _ptr(chosen.weights if chosen else None),
            chosen.ids.shape[1] if chosen else 0, chosen.n_experts if chosen else 0, _ptr(chosen.rows if chosen else None),
            chosen.rows.stride(0) if chosen else 0, _ptr(x32), kind, alpha, _ptr(gain), _ptr(nbias), _ptr(normed),
            normed.stride(0) if normed is not None else 0, n, D, self._stream())
        return x32, normed

    _GATED_ACTS = {"gelu_tanh": 0, "silu": 1, "clamped_swish": 2}

    def gated_act(self, z, hidden: int, act: str, gate_bias=None, up_bias=None, row_scale=None, limit: float = 0.0):
        """act(w * (z[:, :hidden] + gate_bias)) * (w * (z[:, hidden:2 hidden] + up_bias)) in the compute type, w being
        row_scale [rows] (None: 1). z: [rows, >= 2 hidden] 32-bit (a strided view is fine); act: "gelu_tanh", "silu", or
        "clamped_swish": g sigmoid(1.702 g) (u + 1) with g = min(gate, limit) and u = clamp(up, -limit, limit)."""
        n = z.shape[0]
        self._f32_rows(z, "gated_act z", n, 2 * hidden)
        for t, what, size in ((gate_bias, "gate bias", hidden), (up_bias, "up bias", hidden), (row_scale, "row factors", n)):
            if t is not None:
                self._f32(t, "gated_act " + what, size)
        if act not in self._GATED_ACTS:
            raise KernelError(f"gated_act: activation {act!r} (known: {', '.join(self._GATED_ACTS)})")
        out = self.empty(n, hidden)
        self._lazy("stream32").tis_gated_act(self.code, _ptr(z), z.stride(0), int(hidden), _ptr(gate_bias), _ptr(up_bias),
                                             _ptr(row_scale), self._GATED_ACTS[act], _ptr(out), out.stride(0), n,
                                             float(limit), self._stream())
        return out

    _ROW_ACTS = {"gelu_tanh": 0, "silu": 1, "sigmoid": 2, "relu2": 3}

    def activate_rows(self, z, act: str):
        """act(z) in the compute type. z: [rows, W] 32-bit (a strided view is fine); act: "gelu_tanh", "silu", "sigmoid"
        or "relu2" (the square of relu)."""
        _rows_view(self._check(z, "activate_rows z", torch.float32), "activate_rows z")
        if act not in self._ROW_ACTS:
            raise KernelError(f"activate_rows: activation {act!r} (known: {', '.join(self._ROW_ACTS)})")
        n, W = z.shape
        out = self.empty(n, W)
        self._lazy("stream32").tis_activate_rows(self.code, _ptr(z), z.stride(0), self._ROW_ACTS[act], _ptr(out), out.stride(0),
                                                 n, W, self._stream())
        return out

    def normed_mean(self, branches, eps: float):
        """The mean of one or two rows after an RMS norm each: (1 / n) sum_i y_i / sqrt(mean(y_i^2) + eps) * gain_i, in
        32-bit. branches: (y [rows, width] 32-bit (a strided view is fine), gain [width])."""
        if not 1 <= len(branches) <= 2:
            raise KernelError(f"normed_mean: {len(branches)} branches (one or two)")
        n, D = branches[0][0].shape
        for y, gain in branches:
            self._f32_rows(y, "normed_mean branch", n, D)
            self._f32(gain, "normed_mean gain", D)
        (y0, g0), (y1, g1) = branches[0], (branches[1] if len(branches) > 1 else (None, None))
        out = torch.empty(n, D, dtype=torch.float32, device=self.device)
        self._lazy("stream32").tis_normed_mean(_ptr(y0), y0.stride(0), _ptr(g0), _ptr(y1), y1.stride(0) if y1 is not None else 0,
                                               _ptr(g1), float(eps), _ptr(out), n, D, self._stream())
        return out

    _LOWRANK_KINDS = {"sigmoid_root": 0, "exp_softplus": 1, "none": 2}

    def lowrank_act(self, low, w2, bias, kind: str, rate=None, group: int = 1, tau: float = 1.0):
        """The second half of a low-rank projection in 32-bit: act(low . w2^T + bias) with low [rows, rank] (a strided view
        is fine), w2 [channels, rank], bias [channels] or None. kind "sigmoid_root": sigmoid(z)^(1/tau); "exp_softplus":
        exp(-rate[c // group] * softplus(z)), a decay with one rate per run of `group` channels; "none": z."""
        n, rank = low.shape
        _rows_view(self._check(low, "lowrank_act low", torch.float32), "lowrank_act low")
        C = w2.shape[0]
        self._f32(w2, "lowrank_act w2", C * rank)
        if bias is not None:
            self._f32(bias, "lowrank_act bias", C)
        if kind not in self._LOWRANK_KINDS:
            raise KernelError(f"lowrank_act: kind {kind!r} (known: {', '.join(self._LOWRANK_KINDS)})")
        if kind == "exp_softplus":
            if group < 1 or C % group:
                raise KernelError(f"lowrank_act: {C} channels in runs of {group}")
            self._f32(rate, "lowrank_act rates", C // group)
        out = torch.empty(n, C, dtype=torch.float32, device=self.device)
        self._lazy("stream32").tis_lowrank_act(_ptr(low), low.stride(0), rank, _ptr(w2), _ptr(bias), self._LOWRANK_KINDS[kind],
                                               float(tau), _ptr(rate if kind == "exp_softplus" else None), int(group),
                                               _ptr(out), n, C, self._stream())
        return out

    def softcap(self, z, cap: float):
        """z <- cap * tanh(z / cap) on 32-bit rows, in place."""
        _rows_view(self._check(z, "softcap z", torch.float32), "softcap z")
        self._lazy("stream32").tis_softcap(_ptr(z), z.stride(0), float(cap), z.shape[0], z.shape[1], self._stream())
        return z

    # ---- what stands around the scan of a selective state-space mixer ----------------------------------------------
    def conv_prepare(self, proj, xbc_off, dt_off, taps, tap_bias, dt_bias, neg_a, state, conv_at, batch, n_heads, vdim):
        """A short causal convolution with silu over `channels` columns of a 32-bit input product (from xbc_off; the
        first heads * vdim of them are the scan's inputs x), and the step size dt = softplus(proj[:, dt_off + head] +
        dt_bias) per head. Returns u [rows, channels + heads * vdim + heads] 32-bit: the convolved channels, x * dt,
        and exp(neg_a * dt). taps: [channels, taps], the last column weighs the row itself. A row's earlier inputs come
        from the step's rows, and before those from the request's state line (from float conv_at on, [taps - 1]
        [channels], oldest first)."""
        n = proj.shape[0]
        C, K = taps.shape
        inner = n_heads * vdim
        self._f32_rows(proj, "conv_prepare projections", n, max(xbc_off + C, dt_off + n_heads))
        self._f32(taps, "conv taps", C * K)
        if tap_bias is not None:
            self._f32(tap_bias, "conv bias", C)
        self._f32(dt_bias, "dt bias", n_heads)
        self._f32(neg_a, "decay rates", n_heads)
        self._check(state, "state", torch.float32)
        if state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < conv_at + (K - 1) * C:
            raise KernelError(f"conv_prepare: state {tuple(state.shape)} for {(K - 1) * C} floats from {conv_at}")
        self._index(batch.row_seq, "row_seq", n)
        self._index(batch.cu_rows, "cu_rows", batch.n_seqs + 1)
        self._index(batch.seq_slots, "seq_slots", batch.n_seqs)
        if max(batch.host_slots, default=0) >= state.shape[0]:
            raise KernelError(f"conv_prepare: slot {max(batch.host_slots)} of {state.shape[0]}")
        u = torch.empty(n, C + inner + n_heads, dtype=torch.float32, device=self.device)
        self._lazy("ssm_parts").tis_conv_prepare(
            _ptr(proj), proj.stride(0), xbc_off, dt_off, _ptr(taps), _ptr(tap_bias), _ptr(dt_bias), _ptr(neg_a), _ptr(state),
            state.stride(0), conv_at, _ptr(batch.row_seq), _ptr(batch.cu_rows), _ptr(batch.seq_slots), _ptr(u), u.stride(0),
            n, C, K, n_heads, vdim, self._stream())
        return u

    def conv_state_update(self, proj, xbc_off, channels, taps, state, conv_at, batch):
        """Every request's last taps - 1 convolution inputs (columns xbc_off.. of proj, older ones from the line itself
        where the step brings fewer rows) into its state line from float conv_at on."""
        n = proj.shape[0]
        self._f32_rows(proj, "conv_state_update projections", n, xbc_off + channels)
        self._check(state, "state", torch.float32)
        if state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < conv_at + (taps - 1) * channels:
            raise KernelError(f"conv_state_update: state {tuple(state.shape)} for {(taps - 1) * channels} floats from {conv_at}")
        self._index(batch.cu_rows, "cu_rows", batch.n_seqs + 1)
        self._index(batch.seq_slots, "seq_slots", batch.n_seqs)
        if max(batch.host_slots, default=0) >= state.shape[0]:
            raise KernelError(f"conv_state_update: slot {max(batch.host_slots)} of {state.shape[0]}")
        self._lazy("ssm_parts").tis_conv_state_update(_ptr(proj), proj.stride(0), xbc_off, _ptr(state), state.stride(0),
                                                      conv_at, _ptr(batch.cu_rows), _ptr(batch.seq_slots), batch.n_seqs,
                                                      channels, taps, self._stream())

    def gated_group_norm(self, y, x, skip, vdim: int, z, gain, eps: float, parts: int):
        """v = (y + skip[head] * x) * silu(z), each of `parts` equal parts of a row divided by its own root mean square
        (eps under the root), times gain; in the compute type. y, x, z: [rows, width] 32-bit (strided views are fine);
        skip [width / vdim] or None (then x is not read); z None: no gate."""
        n, W = y.shape
        self._f32_rows(y, "gated_group_norm y", n, W)
        if skip is not None:
            self._f32_rows(x, "gated_group_norm x", n, W)
            if W % vdim:
                raise KernelError(f"gated_group_norm: width {W} in heads of {vdim}")
            self._f32(skip, "gated_group_norm skip", W // vdim)
        if z is not None:
            self._f32_rows(z, "gated_group_norm z", n, W)
        self._f32(gain, "gated_group_norm gain", W)
        if parts < 1 or W % parts:
            raise KernelError(f"gated_group_norm: width {W} in {parts} parts")
        out = self.empty(n, W)
        self._lazy("ssm_parts").tis_gated_group_norm(
            self.code, _ptr(y), y.stride(0), _ptr(x if skip is not None else None), x.stride(0) if skip is not None else 0,
            _ptr(skip), int(vdim), _ptr(z), z.stride(0) if z is not None else 0, _ptr(gain), float(eps), _ptr(out),
            out.stride(0), n, W, int(parts), self._stream())
        return out

    # ---- products in groups: experts, heads -----------------------------------------------------------------
    def _grouped(self, a, lda, a_group, a_div, w, c, ldc, c_group, lists, counts, line, most_rows, act=0):
        G, N, K = w.shape
        self._check(w, "grouped product matrices")
        if not w.is_contiguous():
            raise KernelError("grouped product: the matrices must be contiguous [groups, out, in]")
        self._lazy("experts").tis_grouped_linear(
            _DT[a.dtype], _DT[c.dtype], _ptr(a), lda, a_group, a_div, _ptr(w), _ptr(c), ldc, c_group, _ptr(lists),
            _ptr(counts), line, G, most_rows, N, K, act, self._stream())

    def heads_linear(self, x, w, out, out_group: int, out_offset: int = 0):
        """A product per head on the head's own columns: out[:, out_offset + h * out_group + (0..N)] =
        x[:, h * K + (0..K)] . w[h]^T for w [heads, N, K]. x: [rows, heads * K] in the compute type; out: a 2-d tensor
        of the compute type or 32-bit whose other columns are left as they are."""
        _rows_view(self._check(x, "heads_linear x"), "heads_linear x")
        H, N, K = w.shape
        n = x.shape[0]
        if x.shape[1] != H * K:
            raise KernelError(f"heads_linear: x has {x.shape[1]} columns for {H} heads of {K}")
        if out.dtype not in (self.dtype, torch.float32):
            raise KernelError(f"heads_linear: out dtype {out.dtype}")
        _rows_view(self._check(out, "heads_linear out", out.dtype), "heads_linear out")
        if out.shape[0] != n or out_offset < 0 or out_group < N or out_offset + (H - 1) * out_group + N > out.shape[1]:
            raise KernelError(f"heads_linear: out {tuple(out.shape)} for {n} rows, {H} heads of {N} every {out_group} from "
                              f"{out_offset}")
        if n:
            self._grouped(x, x.stride(0), K, 1, w, out[:, out_offset:], out.stride(0), out_group, None, None, 0, n)
        return out

    def route_topk(self, z, correction, scale: float, top: int, score: str = "softmax", groups=None, renorm: bool = False):
        """A router's choice: (ids [rows, top] int32, weights [rows, top] 32-bit). s = softmax(z) over a row's outputs
        (score "sigmoid": sigmoid(z), each output by itself); the `top` outputs with the largest s + correction are
        chosen; an output's weight is s * scale. groups = (count, keep): the outputs form `count` equal runs of
        neighbours, a group's score is its largest s + correction, and only outputs of the `keep` best groups can be
        chosen. renorm: the chosen weights are divided by their sum (+ 1e-20) before the scale."""
        if score not in ("softmax", "sigmoid"):
            raise KernelError(f"route_topk: score {score!r} (known: 'softmax', 'sigmoid')")
        n, E = z.shape
        self._f32_rows(z, "router outputs", n, E)
        if correction is not None:
            self._f32(correction, "router correction", E)
        ids = torch.empty(n, top, dtype=torch.int32, device=self.device)
        weights = torch.empty(n, top, dtype=torch.float32, device=self.device)
        count, keep = (int(groups[0]), int(groups[1])) if groups is not None else (1, 1)
        if count < 1 or E % count or not 1 <= keep <= count or top > keep * (E // count):
            raise KernelError(f"route_topk: {E} outputs in {count} groups of which {keep} are kept, top {top}")
        self._lazy("experts").tis_route_topk(_ptr(z), z.stride(0), _ptr(correction), float(scale), n, E, int(top),
                                             1 if score == "sigmoid" else 0, _ptr(ids), _ptr(weights), count, keep,
                                             1 if renorm else 0, self._stream())
        return ids, weights

    def routed_experts(self, x, ids, weights, w_up, w_down, act: str = "gelu_erf", combine: bool = True):
        """sum_k weights[:, k] * expert(ids[:, k])(x) in 32-bit: expert e < len(w_up) is w_down[e] . act(w_up[e] . x),
        any id beyond is an identity expert whose result is x itself. x: [rows, width] in the compute type; w_up
        [experts, hidden, width], w_down [experts, width, hidden]. combine=False: the experts' results line by
        (row, choice), not summed yet, as a `ChosenExperts` that residual_norm takes in place of a branch."""
        _rows_view(self._check(x, "experts x"), "experts x")
        n, D = x.shape
        top = ids.shape[1]
        E = w_up.shape[0] if w_up is not None else 0
        self._index(ids, "expert ids", n * top)
        self._f32(weights, "expert weights", n * top)
        if act != "gelu_erf":
            raise KernelError(f"routed_experts: activation {act!r} (known: 'gelu_erf')")
        lib = self._lazy("experts")
        y = None
        if E and n:
            F = w_up.shape[1]
            if tuple(w_up.shape) != (E, F, D) or tuple(w_down.shape) != (E, D, F):
                raise KernelError(f"routed_experts: matrices {tuple(w_up.shape)} and {tuple(w_down.shape)} for width {D}")
            lists = torch.empty(E, n, dtype=torch.int32, device=self.device)
            counts = torch.empty(E, dtype=torch.int32, device=self.device)
            lib.tis_expert_lists(_ptr(ids), n * top, E, n, _ptr(lists), _ptr(counts), self._stream())
            hidden = self.empty(n * top, F)
            self._grouped(x, x.stride(0), 0, top, w_up, hidden, hidden.stride(0), 0, lists, counts, n, n, act=1)
            y = torch.empty(n * top, D, dtype=torch.float32, device=self.device)
            self._grouped(hidden, hidden.stride(0), 0, 1, w_down, y, D, 0, lists, counts, n, n)
        if not combine:
            return ChosenExperts(y, ids, weights, E, x)
        out = torch.empty(n, D, dtype=torch.float32, device=self.device)
        lib.tis_experts_combine(self.code, _ptr(y), D, _ptr(x), x.stride(0), _ptr(ids), _ptr(weights), top, E, _ptr(out), D,
                                n, D, self._stream())
        return out

    def gated_experts(self, x, ids, weights, w_gate_up, w_down, act: str = "silu", limit: float = 0.0, weigh: str = "input",
                      n_experts=None):
        """Gated experts whose router weight scales the expert's input: for every (row, choice) the line
        w_down[e] . (act(w * g) * (w * u)) with [g | u] = w_gate_up[e] . x, e = ids[row, choice], w = weights[row,
        choice] (an expert without biases applied to w * x), in 32-bit, not summed: a `ChosenExperts` whose weights are
        None, for a residual sum that adds a row's lines. x: [rows, width] in the compute type; w_gate_up
        [experts, 2 hidden, width] (the gate's rows first), w_down [experts, width, hidden]."""
        _rows_view(self._check(x, "experts x"), "experts x")
        n, D = x.shape
        top = ids.shape[1]
        self._index(ids, "expert ids", n * top)
        self._f32(weights, "expert weights", n * top)
        if weigh not in ("input", "output"):
            raise KernelError(f"gated_experts: weigh {weigh!r} ('input' or 'output')")
        # weigh "output": a chosen expert's weight multiplies its result (in the sum over a row's choices, which the
        # residual sum takes); ids from the number of matrices on are identity experts whose result is the row itself
        if w_gate_up is None:
            if weigh != "output":
                raise KernelError("gated_experts: identity experts alone weigh their results")
            return ChosenExperts(None, ids, weights, 0, x)
        E, F2 = w_gate_up.shape[0], w_gate_up.shape[1]
        F = F2 // 2
        if E < 1 or F2 % 2 or tuple(w_gate_up.shape) != (E, 2 * F, D) or tuple(w_down.shape) != (E, D, F):
            raise KernelError(f"gated_experts: matrices {tuple(w_gate_up.shape)} and {tuple(w_down.shape)} for width {D}")
        y = torch.empty(n * top, D, dtype=torch.float32, device=self.device)
        if weigh == "output":
            if n:
                lists = torch.empty(E, n, dtype=torch.int32, device=self.device)
                counts = torch.empty(E, dtype=torch.int32, device=self.device)
                self._lazy("experts").tis_expert_lists(_ptr(ids), n * top, E, n, _ptr(lists), _ptr(counts), self._stream())
                z = torch.empty(n * top, 2 * F, dtype=torch.float32, device=self.device)
                self._grouped(x, x.stride(0), 0, top, w_gate_up, z, z.stride(0), 0, lists, counts, n, n)
                hidden = self.gated_act(z, F, act, limit=limit)
                self._grouped(hidden, hidden.stride(0), 0, 1, w_down, y, D, 0, lists, counts, n, n)
            return ChosenExperts(y, ids, weights, E, x)
        if n:
            lists = torch.empty(E, n, dtype=torch.int32, device=self.device)
            counts = torch.empty(E, dtype=torch.int32, device=self.device)
            self._lazy("experts").tis_expert_lists(_ptr(ids), n * top, E, n, _ptr(lists), _ptr(counts), self._stream())
            z = torch.empty(n * top, 2 * F, dtype=torch.float32, device=self.device)
            self._grouped(x, x.stride(0), 0, top, w_gate_up, z, z.stride(0), 0, lists, counts, n, n)
            hidden = self.gated_act(z, F, act, row_scale=weights.view(-1))
            self._grouped(hidden, hidden.stride(0), 0, 1, w_down, y, D, 0, lists, counts, n, n)
        return ChosenExperts(y, ids, None, E, x)

    def combine_experts(self, chosen):
        """The sum that a `ChosenExperts` stands for, as 32-bit rows (a block's residual sum usually takes it instead)."""
        n, D = chosen.rows.shape
        return self.residual_norm(torch.zeros(n, D, dtype=torch.float32, device=self.device), chosen)[0]

    # ---- attention with keys and values of different sizes -----------------------------------------------
    def _check_kv_plane(self, plane, n_kv_heads, key_dim, value_dim, page_size):
        self._check(plane, "cache plane")
        per_page = n_kv_heads * page_size * (key_dim + value_dim)
        if not plane.is_contiguous() or plane.shape[0] < 1 or plane.numel() != plane.shape[0] * per_page:
            raise KernelError(f"cache plane {tuple(plane.shape)} does not hold pages of {n_kv_heads} heads x {page_size} "
                              f"slots x ({key_dim} + {value_dim})")

    def attention_prepare(self, proj, q_off, k_off, v_off, positions, write_slots, plane, n_heads, n_kv_heads, key_dim,
                          value_dim, page_size, q_gain=None, k_gain=None, q_factor=None, freqs=None, rot_dims=0, eps=0.0,
                          write_cache=True, value_norm=True, q_bias=None, k_bias=None, v_bias=None, temp_coef=0.0,
                          temp_every=1, whole_norm=False, pair_half=False):
        """From a row's 32-bit projections (queries at column q_off, keys at k_off, values at v_off): queries
        [rows, heads*key_dim] in the compute type; keys and values go into the pages at write_slots. On the way, each
        where its argument is given: biases are added; queries and keys are normed per head (RMS, gain of key_dim
        entries); the first rot_dims channels are rotated in interleaved pairs (angle = position * freqs[pair]);
        queries are multiplied by q_factor[head] and by 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1);
        values are divided by their root mean square (value_norm). whole_norm: the norms run over all heads of a row's
        queries (keys) at once, with gains of heads * key_dim (kv_heads * key_dim) entries. pair_half: the rotated pairs
        are (i, i + rot_dims / 2) instead of (2i, 2i + 1)."""
        n = proj.shape[0]
        need = max(q_off + n_heads * key_dim, k_off + n_kv_heads * key_dim, v_off + n_kv_heads * value_dim)
        self._f32_rows(proj, "attention_prepare projections", n, need)
        self._index(positions, "positions", n)
        for t, what, size in ((q_gain, "query norm gain", n_heads * key_dim if whole_norm else key_dim),
                              (k_gain, "key norm gain", n_kv_heads * key_dim if whole_norm else key_dim),
                              (q_factor, "query factors", n_heads), (q_bias, "query bias", n_heads * key_dim),
                              (k_bias, "key bias", n_kv_heads * key_dim), (v_bias, "value bias", n_kv_heads * value_dim)):
            if t is not None:
                self._f32(t, what, size)
        if rot_dims:
            self._f32(freqs, "rotary frequencies", rot_dims // 2)
        if write_cache:
            self._index(write_slots, "write_slots", n)
            self._check_kv_plane(plane, n_kv_heads, key_dim, value_dim, page_size)
        q = self.empty(n, n_heads * key_dim)
        self._lazy("attention_window").tis_attention_prepare(
            self.code, _ptr(proj), proj.stride(0), q_off, k_off, v_off, _ptr(positions),
            _ptr(write_slots if write_cache else None), _ptr(plane if write_cache else None), _ptr(q), q.stride(0),
            _ptr(q_bias), _ptr(k_bias), _ptr(v_bias), _ptr(q_gain), _ptr(k_gain), _ptr(q_factor),
            _ptr(freqs if rot_dims else None), int(rot_dims), float(eps), 1 if value_norm else 0, float(temp_coef),
            int(temp_every), 1 if whole_norm else 0, 1 if pair_half else 0, n, n_heads, n_kv_heads, key_dim, value_dim,
            page_size, self._stream())
        return q

    def latent_prepare(self, proj, q_off, c_off, positions, write_slots, plane, n_heads, dim, rot_dim, rank, page_size,
                       gain, freqs, rot_dims, eps, write_cache=True):
        """The step before attention over a shared latent. A row's 32-bit projections hold, from column q_off, its
        query heads as [dim unrotated | rot_dim rotated] each, and from c_off the latent (rank channels) followed by
        one rotated key part (rot_dim). Returns (q [rows, heads * (rank + rot_dim)] with every head's rotated part in
        place behind `rank` columns that the caller fills, q_plain [rows, heads * dim]: the unrotated parts), both in
        the compute type. The latent, RMS-normed with `gain`, and the rotated key part go into the pages at
        write_slots as keys of rank + rot_dim channels, and the latent once more as the key's value (pages of one
        key/value head with keys of rank + rot_dim and values of rank channels). Rotation: interleaved pairs of the
        first rot_dims channels of the rotated parts, angle = position * freqs[pair]."""
        n = proj.shape[0]
        self._f32_rows(proj, "latent_prepare projections", n, max(q_off + n_heads * (dim + rot_dim), c_off + rank + rot_dim))
        self._index(positions, "positions", n)
        self._f32(gain, "latent norm gain", rank)
        if rot_dims:
            self._f32(freqs, "rotary frequencies", rot_dims // 2)
        if write_cache:
            self._index(write_slots, "write_slots", n)
            self._check_kv_plane(plane, 1, rank + rot_dim, rank, page_size)
        q = self.empty(n, n_heads * (rank + rot_dim))
        q_plain = self.empty(n, n_heads * max(dim, 1))
        self._lazy("attention_window").tis_latent_prepare(
            self.code, _ptr(proj), proj.stride(0), q_off, c_off, _ptr(positions), _ptr(write_slots if write_cache else None),
            _ptr(plane if write_cache else None), _ptr(q), q.stride(0), _ptr(q_plain), q_plain.stride(0), _ptr(gain),
            _ptr(freqs if rot_dims else None), int(rot_dims), float(eps), n, n_heads, dim, rot_dim, rank, page_size,
            self._stream())
        return q, q_plain

    def plan_latent(self, n_heads: int, seq_rows, add):
        """Host planning for attention over a latent: the items of the matrix-core kernel for a step's rows, (first row,
        rows) each, as many consecutive rows of one request as 16 columns hold heads. Steps of single rows need no list."""
        if self.dtype != torch.bfloat16 or all(n <= 1 for _, _, n in seq_rows):
            return {}
        items = latent_items(seq_rows, n_heads)
        return {("latent_items", n_heads): (add(items), len(items))}

    def latent_attention(self, q, plane, batch, group, n_heads, key_dim, value_dim, page_size, scale):
        """Attention of the rows in `batch` over the pages of a latent: one key/value head, keys of key_dim channels
        whose first value_dim are also kept as values. q: [rows, heads * key_dim]; the result [rows, heads * value_dim].
        bfloat16 with pages of 16 slots, key sizes in steps of 8 and value sizes in steps of 16 run on the matrix cores
        (a library per pair of sizes, compiled when first asked for); anything else on the kernel for any sizes."""
        _rows_view(self._check(q, "q"), "q")
        n = q.shape[0]
        if not (self.dtype == torch.bfloat16 and page_size == 16 and key_dim % 8 == 0 and value_dim % 16 == 0
                and value_dim <= key_dim < 10000 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0):
            return self.paged_attention_kv(q, plane, batch, group, n_heads, 1, key_dim, value_dim, page_size, 0, scale)
        self._check_kv_plane(plane, 1, key_dim, value_dim, page_size)
        if q.shape[1] != n_heads * key_dim:
            raise KernelError(f"attention: q width {q.shape[1]} is not heads {n_heads} x key size {key_dim}")
        tables = batch.block_tables[group]
        self._check(tables, "block tables", torch.int32)
        if tables.dim() != 2 or tables.stride(1) != 1:
            raise KernelError(f"attention: block tables {tuple(tables.shape)} must be 2-d")
        self._index(batch.positions, "positions", n)
        self._index(batch.row_seq, "row_seq", n)
        if batch.max_kv_len > tables.shape[1] * page_size:
            raise KernelError(f"attention: a row sees {batch.max_kv_len} keys but block tables cover "
                              f"{tables.shape[1] * page_size}")
        out = self.empty(n, n_heads * value_dim)
        if n == 0:
            return out
        items, n_items = None, n
        if batch.max_seq_rows > 1:
            plan = batch.extras.get(("latent_items", n_heads))
            if plan is None:        # a caller that did not plan (a kernel test)
                host = latent_items(batch.seq_rows, n_heads)
                plan = (torch.from_numpy(host).reshape(-1).to(self.device), len(host))
            items, n_items = plan[0].reshape(-1), plan[1]
            if items.numel() < 2 * n_items or items.dtype != torch.int32 or not items.is_contiguous():
                raise KernelError(f"attention: a list of {items.numel()} integers for {n_items} items")
        # Portions: the four-wave kernel, every item's keys whole. Single rows: a wave per row and 16 heads, with
        # enough waves to fill the chip: a request's keys are cut where its rows alone would leave most units idle
        waves = n_items * -(-n_heads // 16)
        steps = -(-batch.max_kv_len // 32)
        most = max(1, (self._workspace.numel() // (n * n_heads * (value_dim + 2))))
        # (a wave's step is two or three dependent trips to memory and little else, so many short chains beat few long
        # ones: four waves a compute unit, down to one step each)
        n_splits = 0 if items is not None else int(max(1, min(-(-4 * self.units // waves), steps, 64, most)))
        part_o = part_ml = None
        if n_splits > 1:
            part_o = self._workspace
            part_ml = self._workspace[n * n_heads * n_splits * value_dim:]
        lib = self._lazy(f"attention_latent@{key_dim * 10000 + value_dim}")
        lib.tis_attention_latent(_ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0), _ptr(batch.row_seq),
                                 _ptr(batch.positions), _ptr(items), n_items, _ptr(out), out.stride(0), _ptr(part_o),
                                 _ptr(part_ml), n, n_heads, key_dim, value_dim, page_size, float(scale), n_splits,
                                 self._stream())
        return out

    def paged_attention_kv(self, q, plane, batch, group, n_heads, n_kv_heads, key_dim, value_dim, page_size, window=0,
                           scale=None, sink=False, gate=None, chunk=0):
        """Attention of the rows in `batch` over pages whose keys have key_dim and whose values value_dim channels:
        [rows, heads*value_dim]. chunk > 0: a row at position p sees only the keys from p - p % chunk on (its own chunk
        of positions; a chunk's edges are multiples of `chunk` in the request). sink: the softmax's denominator also counts a key of score 0 that has no value.
        gate: [rows, heads] 32-bit (a strided view is fine); head h's result is multiplied by sigmoid(gate[:, h])."""
        _rows_view(self._check(q, "q"), "q")
        n = q.shape[0]
        self._check_kv_plane(plane, n_kv_heads, key_dim, value_dim, page_size)
        if q.shape[1] != n_heads * key_dim:
            raise KernelError(f"attention: q width {q.shape[1]} is not heads {n_heads} x key size {key_dim}")
        if gate is not None:
            self._f32_rows(gate, "attention gate", n, n_heads)
        tables = batch.block_tables[group]
        self._check(tables, "block tables", torch.int32)
        if tables.dim() != 2 or tables.stride(1) != 1:
            raise KernelError(f"attention: block tables {tuple(tables.shape)} must be 2-d")
        self._index(batch.positions, "positions", n)
        self._index(batch.row_seq, "row_seq", n)
        if batch.max_kv_len > tables.shape[1] * page_size:
            raise KernelError(f"attention: a row sees {batch.max_kv_len} keys but block tables cover "
                              f"{tables.shape[1] * page_size}")
        out = self.empty(n, n_heads * value_dim)
        self._lazy("attention_window").tis_attention_window(
            self.code, _ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0), _ptr(batch.row_seq),
            _ptr(batch.positions), _ptr(out), out.stride(0), n, n_heads, n_kv_heads, key_dim, value_dim, page_size,
            int(window), int(chunk), float(scale if scale is not None else key_dim ** -0.5), 1 if sink else 0, _ptr(gate),
            gate.stride(0) if gate is not None else 0, self._stream())
        return out

    def plan_row_tiles(self, seq_rows, add):
        """Host planning for the matrix-core attention with mixed sigmoid weights: its items for a step's rows, (first
        row, rows) each, up to 16 consecutive rows of one request. Steps of single rows need no list."""
        if self.dtype != torch.bfloat16 or all(n <= 1 for _, _, n in seq_rows):
            return {}
        items = latent_items(seq_rows, 1, 16)
        return {("row_tiles", 16): (add(items), len(items))}

    def _mixed_on_matrix_cores(self, q, key_dim, value_dim, page_size, n_heads):
        return (self.dtype == torch.bfloat16 and page_size == 16 and key_dim % 8 == 0 and value_dim % 16 == 0
                and key_dim <= 512 and value_dim <= 512 and n_heads <= 28 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0
                and -(-n_heads // 4) * (value_dim // 16 + key_dim // 32) <= 64)

    def mixed_sigmoid_attention(self, q, plane, batch, group, n_heads, n_kv_heads, key_dim, value_dim, page_size, chunk,
                                scale, softcap, head_bias, talk):
        """Attention of the rows in `batch` whose weights are sigmoids mixed across the heads: for every key j that the
        row at position p sees (j <= p; chunk > 0: only from p - p % chunk on), w_g = sigmoid(cap(q_g . k * scale) +
        head_bias[g]) with cap(s) = softcap * tanh(s / softcap) (softcap 0: s), head h weighs the values of its own
        key/value head with sum_g talk[h, g] * w_g. Nothing is normalised over the keys. [rows, heads * value_dim]."""
        _rows_view(self._check(q, "q"), "q")
        n = q.shape[0]
        self._check_kv_plane(plane, n_kv_heads, key_dim, value_dim, page_size)
        if q.shape[1] != n_heads * key_dim:
            raise KernelError(f"attention: q width {q.shape[1]} is not heads {n_heads} x key size {key_dim}")
        self._f32(head_bias, "attention head bias", n_heads)
        self._f32(talk, "attention head mixture", n_heads * n_heads)
        tables = batch.block_tables[group]
        self._check(tables, "block tables", torch.int32)
        if tables.dim() != 2 or tables.stride(1) != 1:
            raise KernelError(f"attention: block tables {tuple(tables.shape)} must be 2-d")
        self._index(batch.positions, "positions", n)
        self._index(batch.row_seq, "row_seq", n)
        if batch.max_kv_len > tables.shape[1] * page_size:
            raise KernelError(f"attention: a row sees {batch.max_kv_len} keys but block tables cover "
                              f"{tables.shape[1] * page_size}")
        out = self.empty(n, n_heads * value_dim)
        if n == 0:
            return out
        longest = min(batch.max_kv_len, chunk) if chunk > 0 else batch.max_kv_len
        if self._mixed_on_matrix_cores(q, key_dim, value_dim, page_size, n_heads):
            # bfloat16 with pages of 16 slots: four waves an item of up to 16 rows, a library per sizes (compiled when a
            # model first asks for it)
            items, n_items = None, n
            if batch.max_seq_rows > 1:
                plan = batch.extras.get(("row_tiles", 16))
                if plan is None:        # a caller that did not plan (a kernel test)
                    host = latent_items(batch.seq_rows, 1, 16)
                    plan = (torch.from_numpy(host).reshape(-1).to(self.device), len(host))
                items, n_items = plan[0].reshape(-1), plan[1]
                if items.numel() < 2 * n_items or items.dtype != torch.int32 or not items.is_contiguous():
                    raise KernelError(f"attention: a list of {items.numel()} integers for {n_items} items")
            # few items: an item's keys are cut over several workgroups (two a compute unit), whose parts are added up
            most = max(1, self._workspace.numel() // (n * n_heads * value_dim))
            n_splits = int(max(1, min(-(-(longest + 31) // 32), (2 * self.units) // n_items, 64, most)))
            hpw = -(-n_heads // 4)
            lib = self._lazy(f"attention_mixed@{key_dim * 100000 + value_dim * 100 + hpw}")
            lib.tis_attention_mixed_mfma(
                _ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0), _ptr(batch.row_seq), _ptr(batch.positions),
                _ptr(items), n_items, _ptr(out), out.stride(0), _ptr(self._workspace if n_splits > 1 else None), n_splits, n,
                n_heads, n_kv_heads, key_dim, value_dim, page_size, int(chunk), float(scale), float(softcap), _ptr(head_bias),
                _ptr(talk), self._stream())
            return out
        # keys a workgroup takes at a time: what LDS holds beside the row's queries, in whole pages
        room = (16384 - n_heads * key_dim - n_heads * n_heads) // (2 * n_heads)
        block = min(256, room // 16 * 16 if room >= 16 else room)
        if block < 1:
            raise KernelError(f"attention: {n_heads} heads of {key_dim} channels do not fit the kernel for any sizes")
        # few rows: a row's keys are cut over several workgroups, whose parts a second kernel adds up
        n_splits = int(max(1, min(-(-longest // block), (2 * self.units) // n, 64)))
        partial = None
        if n_splits > 1:
            need = n * n_splits * n_heads * value_dim
            # (the fixed workspace where there is one and it is large enough; an allocation made while a graph is
            # captured stays with the graph)
            fits = self._workspace is not None and self._workspace.numel() >= need
            partial = self._workspace if fits else torch.empty(need, dtype=torch.float32, device=self.device)
        self._lazy("attention_window").tis_attention_mixed(
            self.code, _ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0), _ptr(batch.row_seq),
            _ptr(batch.positions), _ptr(out), out.stride(0), _ptr(partial), n_splits, n, n_heads, n_kv_heads, key_dim,
            value_dim, page_size, int(chunk), float(scale), float(softcap), _ptr(head_bias), _ptr(talk), int(block),
            self._stream())
        return out

    # ---- a gated delta rule ----------------------------------------------------------------------------------
    def _check_lines(self, what, state, floats, batch):
        self._check(state, "state", torch.float32)
        if state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < floats:
            raise KernelError(f"{what}: state {tuple(state.shape)} for lines of {floats} floats")
        self._index(batch.cu_rows, "cu_rows", batch.n_seqs + 1)
        self._index(batch.seq_slots, "seq_slots", batch.n_seqs)
        if max(batch.host_slots, default=0) >= state.shape[0]:
            raise KernelError(f"{what}: slot {max(batch.host_slots)} of {state.shape[0]}")

    def delta_prepare(self, proj, conv_off, beta_off, taps, state, conv_at, batch, n_heads, qk_heads, dim, vdim):
        """The step before a delta rule's walk, from a row's 32-bit projections: the columns conv_off.. hold q and k
        (qk_heads * dim each) and v (heads * vdim), which go channel by channel through a short causal convolution
        (taps [channels, taps], the last column weighs the row itself; earlier inputs come from the step's rows and
        before those from the request's state line, from float conv_at on, [taps - 1][channels], oldest first) and silu;
        q and k become unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q times dim^(-1/2). Returns
        u [rows, channels + heads] 32-bit: q, k, v, and beta = sigmoid(proj[:, beta_off + head])."""
        n = proj.shape[0]
        C, K = taps.shape
        if C != 2 * qk_heads * dim + n_heads * vdim:
            raise KernelError(f"delta_prepare: {C} convolved channels for {qk_heads} x {dim} q and k and {n_heads} x {vdim} v")
        self._f32_rows(proj, "delta_prepare projections", n, max(conv_off + C, beta_off + n_heads))
        self._f32(taps, "conv taps", C * K)
        self._check_lines("delta_prepare", state, conv_at + (K - 1) * C, batch)
        self._index(batch.row_seq, "row_seq", n)
        u = torch.empty(n, C + n_heads, dtype=torch.float32, device=self.device)
        self._lazy("delta_rule").tis_delta_prepare(
            _ptr(proj), proj.stride(0), int(conv_off), int(beta_off), _ptr(taps), K, _ptr(state), state.stride(0), int(conv_at),
            _ptr(batch.row_seq), _ptr(batch.cu_rows), _ptr(batch.seq_slots), _ptr(u), u.stride(0), n, n_heads, qk_heads, dim,
            vdim, self._stream())
        return u

    def delta_scan(self, u, q_off, k_off, v_off, beta_off, decay, state, batch, n_heads, qk_heads, dim, vdim):
        """Walk the step's rows of every request through its matrix state, in order: per head S <- diag(decay) S;
        w = beta (v - S^T k); S <- S + k w^T; o = S^T q. Returns o [rows, heads * vdim] 32-bit. u: [rows, ...] 32-bit with
        q and k (qk_heads * dim each; head h reads those of qk head h // (heads / qk_heads)), v (heads * vdim) and beta
        (heads) at the given columns; decay [rows, heads * dim]; state: [slots, floats] 32-bit, a line starting with S as
        [heads, blocks of 16 value channels, dim, 16] (lines 16 bytes aligned)."""
        n = u.shape[0]
        self._f32_rows(u, "delta_scan rows", n, max(q_off + qk_heads * dim, k_off + qk_heads * dim, v_off + n_heads * vdim,
                                                    beta_off + n_heads))
        self._f32_rows(decay, "delta_scan decays", n, n_heads * dim)
        self._check_lines("delta_scan", state, n_heads * -(-vdim // 16) * dim * 16, batch)
        if state.stride(0) % 4 or state.data_ptr() % 16:
            raise KernelError("delta_scan: state lines must be 16 bytes aligned")
        out = torch.empty(n, n_heads * vdim, dtype=torch.float32, device=self.device)
        self._lazy("delta_rule").tis_delta_scan(
            _ptr(u), u.stride(0), int(q_off), int(k_off), int(v_off), int(beta_off), _ptr(decay), decay.stride(0), _ptr(state),
            state.stride(0), _ptr(batch.cu_rows), _ptr(batch.seq_slots), batch.n_seqs, _ptr(out), out.stride(0), n_heads,
            qk_heads, dim, vdim, self._stream())
        return out

    # ---- recurrent mixers with a matrix state per head ---------------------------------------------------
    @staticmethod
    def state_scan_floats(kind: str, n_heads: int, dim: int, vdim: int) -> int:
        """32-bit floats of one request's state: S [heads, dim, vdim]; "gated_max" also keeps its normaliser n [dim]
        and running maximum per head, once per block of 16 value channels (the kernel's workgroups)."""
        blocks = -(-vdim // 16)
        return n_heads * dim * vdim + (n_heads * blocks * (dim + 1) if kind == "gated_max" else 0)

    def state_scan(self, kind, proj, q_off, k_off, v_off, q_scale, state, batch, n_heads, dim, vdim, decay=None,
                   i_off=0, f_off=0, bias_i=None, bias_f=None, cap=0.0, qk_group=1, decay_per_head=False):
        """Walk the step's rows of every request through its matrix state, in order, and return o [rows, heads*vdim]
        in 32-bit. kind "decay": S = diag(decay) S + k v^T, o = S^T q. kind "gated_max": scalar log gates per head
        from the columns i_off, f_off of proj (plus biases, capped by cap * tanh(. / cap)), stabilised by a running
        maximum, o normalised by max(|n . q|, exp(-m)) + 1e-6. state: [slots, floats] 32-bit, a line per request.

        qk_group: that many consecutive heads share one set of query and key columns (proj then holds heads / qk_group
        of them). decay_per_head: `decay` holds one number per head and row instead of one per key channel.

        A step whose longest portion has at least two segments' rows (self.scan_segment, 64) is run in segments side
        by side, with a second pass for the states at the segments' starts and a third for what they add to the
        rows' outputs; shorter portions and single tokens are walked in order by one kernel."""
        n = proj.shape[0]
        if qk_group < 1 or n_heads % qk_group:
            raise KernelError(f"state_scan: {n_heads} heads in groups of {qk_group}")
        n_qk = n_heads // qk_group
        need = max(q_off + n_qk * dim, k_off + n_qk * dim, v_off + n_heads * vdim)
        if kind == "gated_max":
            need = max(need, i_off + n_heads, f_off + n_heads)
            self._f32(bias_i, "input gate bias", n_heads)
            self._f32(bias_f, "forget gate bias", n_heads)
        elif kind == "decay":
            self._f32_rows(decay, "decays", n, n_heads if decay_per_head else n_heads * dim)
        else:
            raise KernelError(f"state_scan: unknown kind {kind!r}")
        self._f32_rows(proj, "state_scan projections", n, need)
        self._check(state, "state", torch.float32)
        if state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < self.state_scan_floats(kind, n_heads, dim, vdim):
            raise KernelError(f"state_scan: state {tuple(state.shape)} for lines of "
                              f"{self.state_scan_floats(kind, n_heads, dim, vdim)} floats")
        self._index(batch.cu_rows, "cu_rows", batch.n_seqs + 1)
        self._index(batch.seq_slots, "seq_slots", batch.n_seqs)
        if max(batch.host_slots, default=0) >= state.shape[0]:
            raise KernelError(f"state_scan: slot {max(batch.host_slots)} of {state.shape[0]}")
        out = torch.empty(n, n_heads * vdim, dtype=torch.float32, device=self.device)
        lib = self._lazy("state_scan")
        seg_len = int(getattr(self, "scan_segment", 64))
        segments, workspace = 0, None
        if seg_len > 0 and batch.max_seq_rows >= 2 * seg_len and lib.cdll.tis_state_scan_segmentable(dim):
            segments = -(-batch.max_seq_rows // seg_len)
            lib.cdll.tis_state_scan_workspace.restype = c_long
            floats = lib.cdll.tis_state_scan_workspace(0 if kind == "decay" else 1, batch.n_seqs, segments, n, n_heads,
                                                       dim, vdim)
            workspace = torch.empty(floats, dtype=torch.float32, device=self.device)
        lib.tis_state_scan(
            0 if kind == "decay" else 1, _ptr(proj), proj.stride(0), q_off, k_off, v_off, float(q_scale), _ptr(decay),
            decay.stride(0) if decay is not None else 0, i_off, f_off, _ptr(bias_i), _ptr(bias_f), float(cap),
            _ptr(state), state.stride(0), _ptr(batch.cu_rows), _ptr(batch.seq_slots), batch.n_seqs, _ptr(out),
            out.stride(0), n_heads, dim, vdim, segments, seg_len, n, _ptr(workspace), int(qk_group),
            1 if decay_per_head else 0, self._stream())
        return out

    # ---- sampling ------------------------------------------------------------------------------------
    def argmax(self, logits):
        _rows_view(self._check(logits, "logits", torch.float32), "logits")
        n, V = logits.shape
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        self.sampling.tis_argmax(_ptr(logits), logits.stride(0), n, V, _ptr(out), self._stream())
        return out

    def sample(self, logits, temperature, top_k, top_p, rep_penalty, uniform, ctx_tokens=None, ctx_offsets=None,
               seen=None, seen_row=None):
        """One token per row of 32-bit logits; per-row parameters are device tensors of length rows.

        A request's context for the repetition penalty comes as a flat token list with offsets, or as `seen`, a
        [requests, vocab] byte table (nonzero: occurred) with `seen_row[i]` naming row i's line (-1: none); the
        kernel then also marks the token it draws.
        """
        _rows_view(self._check(logits, "logits", torch.float32), "logits")
        n, V = logits.shape
        for t, what, dt in ((temperature, "temperature", torch.float32), (top_p, "top_p", torch.float32),
                            (uniform, "uniform", torch.float32), (top_k, "top_k", torch.int32)):
            self._check(t, what, dt)
            if t.numel() != n or not t.is_contiguous():
                raise KernelError(f"sample: {what} has {t.numel()} entries for {n} rows")
        if rep_penalty is not None:
            self._check(rep_penalty, "rep_penalty", torch.float32)
            if rep_penalty.numel() != n:
                raise KernelError(f"sample: rep_penalty has {rep_penalty.numel()} entries for {n} rows")
        if ctx_tokens is not None:
            self._index(ctx_tokens, "ctx_tokens")
            self._index(ctx_offsets, "ctx_offsets", n + 1)
        if seen is not None:
            self._check(seen, "seen", torch.uint8)
            if seen.dim() != 2 or seen.shape[1] != V or seen.stride(1) != 1:
                raise KernelError(f"sample: seen {tuple(seen.shape)} is not [requests, {V}]")
            self._index(seen_row, "seen_row", n)
        work = torch.empty(n, V, dtype=torch.float32, device=self.device)
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        self.sampling.tis_sample(_ptr(logits), logits.stride(0), _ptr(work), n, V, _ptr(temperature), _ptr(top_k),
                                 _ptr(top_p), _ptr(rep_penalty), _ptr(ctx_tokens), _ptr(ctx_offsets), _ptr(uniform),
                                 _ptr(out), _ptr(seen), seen.stride(0) if seen is not None else 0,
                                 _ptr(seen_row if seen is not None else None), self._stream())
        return out
