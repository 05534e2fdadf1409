"""Which kernel multiplies a few rows of bfloat16 activations by a bfloat16 matrix.

Pure functions of the shape: they touch no tensor and run anywhere, so the choices can be
tested without a GPU.  Every figure below was measured on one MI355X, under a graph, over 36
different matrices in turn (so that none came from a cache).

Three kernels take part.  ``rows`` (``gemm_rows``): both operands go through LDS in whole
256-byte row segments, the rows of x are shared by a workgroup, K may be cut over workgroups.
``skinny`` (``gemm_skinny``): the earlier one, whose waves split K and read x in the shape of
a matrix-instruction operand.  ``library``: the library's tiled product.  Up to 64 rows the
product is bound by moving the matrix once, and by what a compute unit can pull: the first
kernel wins almost everywhere; the exceptions are listed where they are decided.
"""
from __future__ import annotations

from dataclasses import dataclass

FEW_ROWS = 16      # one tile of rows of x
STREAM_ROWS = 64   # most rows of x a workgroup of a weight-streaming kernel takes
SPLIT_ROWS = 128   # most rows the rows kernel takes as two halves, each to workgroups of its own
TALL = 32768       # a matrix of at least this many rows (a vocabulary head) is "tall"
UNITS = 256        # compute units of an MI355X; callers on a device pass its own count


@dataclass(frozen=True)
class Product:
    """``kernel``: "rows", "skinny" or "library"; ``parts``: ranges K is cut into (each a float
    partial result for the consumer to add); ``col_tiles``: tiles of 16 columns per wave of
    the rows kernel."""
    kernel: str
    parts: int = 1
    col_tiles: int = 1


def aliased_rows(k: int) -> bool:
    """Rows of a power-of-two length of 8 KB or more: the 256-byte segments that a chunk is of
    many rows then meet in few memory channels, and the rows kernel streams 10 to 20 % slower
    (gate/up 2x12288 x 4096 at 8 rows: 44 us against the skinny kernel's 40)."""
    return k % 4096 == 0


def gated_row_padding(k: int, element_size: int) -> int:
    """Elements to leave unused behind every row of a fused gate/up matrix of 16-bit elements
    (of rows of at least 1,024 of them).
    A workgroup's gate rows and its up rows, half the matrix further, otherwise tend to meet in
    the same memory channels, most of all where a row is a power-of-two length of 8 KB or more:
    2x12288 x 4096: the rows kernel at 8 rows 43.0 -> 34.7 us (which then beats the skinny
    kernel's 37.4), at 64 rows 47.3 -> 39.3.  At other widths the streaming kernels gain little
    (2x9728 x 2560 at 8 rows 20.1 -> 19.5 us) and the library's product for prompt portions some
    (2,048 rows of 2x9728 x 2560: 212 -> 187 us alone, 0.2 ms of a 19.8 ms step): a whole step
    at the Qwen3-4B shape 2.526 -> 2.516 ms decoding and 19.81 -> 19.60 ms for 2,048 prompt tokens,
    old and new in turn on one device, three times.  The other products are within 1 % either
    way and stay as they are; 192 elements do no better than 64."""
    return 64 if element_size == 2 and k >= 1024 else 0  # not worth doubling a toy's matrix


def rows_split(n: int, k: int, rows: int = STREAM_ROWS, units: int = UNITS) -> tuple:
    """(parts, col_tiles) of the rows kernel for a product into the residual stream.
    Workgroups of 128 columns for deep matrices (beyond 16 rows, where the rows of x weigh
    more, from a depth of 8192) and for wide ones, else of 64; K cut into the largest power of
    two of parts (at most 16, of at least 256 elements each) that keeps the workgroups at one
    per compute unit or fewer: more of them only re-read the rows of x.  (The kernel then gives
    every workgroup the same share of the columns, so that the launch fills whole rounds of the
    units, where the share stays at least as many rows of w as there are rows of x.)"""
    col_tiles = 2 if (k >= 8192 and rows > FEW_ROWS) or k >= 16384 or n > 4096 else 1
    groups = -(-n // (64 * col_tiles))
    parts = 1
    while parts < 16 and 2 * parts * groups <= units and k // (2 * parts) >= 256:
        parts *= 2
    return parts, col_tiles


def skinny_parts(n: int, k: int, units: int = UNITS) -> int:
    """Ranges the skinny kernel cuts K into so that a matrix of few rows still fills the chip
    (at most 4: with 8 a whole decode step measured 7 % slower)."""
    tiles = (n + 15) // 16
    parts = 1
    while tiles * parts < 2 * units and parts < 4 and k // (parts * 2) >= 512:
        parts *= 2
    return parts


def deep_or_narrow(n: int, k: int) -> bool:
    """Matrices much deeper than wide (a down projection) and those of few rows (an out
    projection)."""
    return k >= 2 * n or n <= 4096


def plan_residual(rows: int, n: int, k: int, units: int = UNITS) -> Product:
    """A product about to be added to the float32 residual stream (out and down projections),
    ``rows`` <= 128: float32 sums, never rounded, from whichever kernel.

    Up to 16 rows the rows kernel beats the skinny one for deep, narrow and moderately wide
    matrices (2560x4096 at 8 rows: 6.2 against 8.3 us, 2560x9728 11.5 against 13.8, 5120x8192
    20 against 23, 5120x25600 52 against 65).  From 17 to 64 rows the rows kernel with K cut
    into parts beats the library, which does not cut K (at 64 rows: 2560x4096 10.0 against
    14.3 us, 2560x9728 16.0 against 28.0, 4096x4096 11.0 against 15.1, 4096x12288 26.5 against
    37.5, 5120x5120 16.3 against 21.8, 5120x8192 22.9 against 28.9, 5120x17408 42 against 86,
    6144x6144 21.5 against 26.8, 10240x10240 48 against 60), except for wide matrices whose rows
    are of a power-of-two length (8192x8192 36.4 against 33.7, 16384x4096 37.4 against 34.5).
    From 65 to 128 rows the rows kernel takes the rows as two halves, each to workgroups of its
    own, two that stream the same rows of w side by side on one die: 2560x9728 at 65, 96 and 128
    rows 22.6, 23.0 and 26.2 us against the library's 26.2, 26.9 and 52.9 (bfloat16 result),
    2560x4096 14.1, 14.3 and 16.8 against 20.9, 20.9 and 22.9; the same choices as for 64 rows."""
    few = rows <= FEW_ROWS
    if few:
        if deep_or_narrow(n, k) or n <= 8192:
            return Product("rows", *rows_split(n, k, rows, units))
        return Product("skinny", skinny_parts(n, k, units))
    if aliased_rows(k) and n >= 8192:
        return Product("library")
    return Product("rows", *rows_split(n, k, rows, units))


def plan_projection(rows: int, n: int, k: int) -> Product:
    """Any other product (q/k/v; the vocabulary head); beyond 64 rows the library's.

    A head (tall matrix): the rows kernel with 128 columns per workgroup (151936 x 2560: 137 us
    against the skinny kernel's 154 at 8 rows; 173 against the library's 186 at 64 rows, 150
    against 173 at 32; x 5120: 264 against 304 and 303 against 313).  With aliased rows (x 4096)
    64 columns per workgroup do better (220 against 227 us at 1 row, 230 against 235 at 8, 262
    against 272 at 32, the skinny kernel 237, 234 and, at 16 rows, 258 against 239), and beyond
    32 rows the library (274 against 286 and 300 at 64 rows).
    A projection up to 16 rows: the rows kernel (6144 x 2560 at 8 rows 9.3 against the skinny
    kernel's 10.7 us, 10240 x 5120 21 against 31, 6144 x 4096 14.5 against 16).  Beyond 16
    rows the library: without K cut over workgroups the rows kernel is within 10 % of it either
    way (6144 x 2560: 12.2 against 11.8 us at 32 rows, 17.8 against 15.5 at 64), and the rows of
    x of a workgroup that covers 64 of many columns weigh most here; a consumer that adds
    partial sums gets them (:func:`plan_summed_later`)."""
    few = rows <= FEW_ROWS
    if rows > STREAM_ROWS:
        return Product("library")
    if n >= TALL:
        if aliased_rows(k):
            return Product("rows", 1, 1) if rows <= 32 else Product("library")
        return Product("rows", 1, 2)
    return Product("rows") if few else Product("library")


def plan_summed_later(rows: int, n: int, k: int, units: int = UNITS) -> Product:
    """A projection whose consumer can add float partial sums itself (q/k/v in front of the
    decode attention that prepares its own operands): K is cut over workgroups where the uncut
    launch would leave compute units without one.

    Up to 16 rows: workgroups of 64 columns and 2 or 4 parts, as many as keep the workgroups
    within the units.  At 8 rows 6144 x 2560 takes 7.8 us (2 parts) against 10.3 uncut, 4096 x
    2048 5.5 (4) against 8.5, 6144 x 4096 12.3 (2) against 14.5, 7168 x 5120 15.0 (2) against
    17.6; 10240 x 5120 stays uncut (19.8 against 20.1).  With what the attention kernel then
    pays for adding them, a whole step at the Qwen3-4B shape, batch 8: 2.603 -> 2.531 ms.
    From 17 to 64 rows the rows kernel so cut beats the library, which does not cut K: 6144 x
    2560 at 17, 32, 48 and 64 rows 9.0, 9.5, 10.8 and 11.7 us (four parts of 128 columns) against
    11.0, 11.8, 15.3 and 15.5; 6144 x 4096 11.8 to 14.9 against 14.5 to 17.9; 10240 x 5120 (two
    parts) 21.5 to 28.1 against 24.4 to 32.8.  From 65 to 128 rows, as two halves: 6144 x 2560 15.4 to
    18.2 us against the library's 20.9 to 21.3.  Without a cut as :func:`plan_projection`."""
    if n < TALL and rows <= FEW_ROWS:
        groups, parts = -(-n // 64), 1
        while parts < 4 and 2 * parts * groups <= units and k // (2 * parts) >= 256:
            parts *= 2
        if parts > 1:
            return Product("rows", parts, 1)
    elif n < TALL and rows <= SPLIT_ROWS:
        parts, col_tiles = rows_split(n, k, rows, units)
        if parts > 1:
            return Product("rows", parts, col_tiles)
    return plan_projection(rows, n, k)


def plan_gated(rows: int, n_half: int, k: int, row_stride: int) -> Product:
    """``silu(x gate^T) * (x up^T)`` over a fused matrix of ``2 * n_half`` rows; "library" means
    its product followed by the activation kernel (up to 64 rows its float32 result).

    Against the skinny kernel at 8 rows: 2x9728 x 2560 20 against 25 us, 2x25600 x 5120 90
    against 105, 2x17408 x 5120 63 against 76, 2x6144 x 2048 13.8 against 15.2; but 2x12288 x
    4096 44 against 39 (aliased rows; with the rows :func:`gated_row_padding` apart in memory
    34.7 against 37.4) and 2x3072 x 1024 7.4 against 6.1 (a small matrix).
    Against the library and the activation kernel from 17 to 64 rows: 2x9728 x 2560 21 to 27
    against 30 to 34, 2x12288 x 4096 45 to 48 against 48 to 53, 2x17408 x 5120 67 to 86 against
    78 to 93, 2x25600 x 5120 91 to 105 against 94 to 107, 2x3072 x 1024 9.3 to 12.8 against
    13.8 to 14.3 (2x6144 x 2048 at 64 rows alone loses, 20.9 against 19.8).  A workgroup of the
    rows kernel sees its gate rows and, ``n_half`` rows further, its up rows through one
    descriptor, which spans at most 2 GB."""
    if rows > STREAM_ROWS:  # 2x9728 x 2560 at 65 to 128 rows: 41 to 48 us against the library's 36 to 38
        return Product("library")
    few = rows <= FEW_ROWS
    fits = (n_half + 64) * row_stride * 2 < 2 ** 31
    if fits and (not few or (not aliased_rows(row_stride) and n_half >= 4096)):
        return Product("rows", 1, 2)
    return Product("skinny") if few else Product("library")
