"""Every matrix product a step of the published Qwen3 dense sizes runs, at its real size,
through the dispatchers the parts call (``ops.linear``, ``ops.linear_for_residual``,
``ops.linear_glu``), against a float64 product: which kernel the plan picks for the case,
how that kernel is laid over the chip, and the numbers.

The vocabulary head is /root/reference/src/pylon/model/model.py:140-144, q/k/v and the out
projection /root/reference/src/pylon/model/layers.py:126,138, gate/up and down :26-27.

Kernel instance reached per case (``gemm_rows_kernel<MT, CT, GLU, WAVES, TO>`` with MT =
ceil(rows / 16); ``groups x parts`` workgroups of ``c`` columns each: every workgroup of a
launch gets the same share of the columns, a whole number of rounds over the 256 compute
units, unless that would make it re-read more rows of x than it streams rows of w):

=========  ========================  =====================================  ===================
product    1, 8, 16 rows             17, 48, 64 rows                        130 rows
=========  ========================  =====================================  ===================
4b qkv     rows CT1 2w 256x1 c24     library, bfloat16                      library, bfloat16
4b out     rows CT1 4w 64x4 c40      rows CT1 4w 64x4 c40 at 17 rows,       library, bfloat16
                                     40x4 c64 at 48 and 64
4b gate/up rows GLU 4w 256x1 c38     rows GLU 4w 256x1 c38                  library + silu_gate
4b down    rows CT1 4w 64x4 c40      rows CT2 4w 32x8 c80                   library, bfloat16
4b head    rows CT2 4w 1277x1 c119   rows CT2 4w 1187x1 c128                library, float32
8b qkv     rows CT1 2w 256x1 c24     library                                library
8b out     rows CT1 4w 64x4 c64      rows CT1 4w 64x4 c64                   library
8b gate/up skinny GLU                rows GLU 4w 256x1 c48                  library + silu_gate
8b down    rows CT1 4w 64x4 c64      rows CT2 4w 32x8 c128                  library
8b head    rows CT1 4w 2533x1 c60    rows CT1 4w 2374x1 c64 at 17 rows,     library, float32
                                     library float32 at 48 and 64
32b qkv    rows CT1 4w 256x1 c40     library                                library
32b out    rows CT2 4w 64x4 c80      rows CT2 4w 64x4 c80                   library
32b g/u    rows GLU 4w 512x1 c50     rows GLU 4w 512x1 c50                  library + silu_gate
32b down   rows CT2 4w 64x4 c80      rows CT2 4w 64x4 c80                   library
32b head   rows CT2 4w 1277x1 c119   rows CT2 4w 1187x1 c128                library, float32
=========  ========================  =====================================  ===================

In front of the decode attention that prepares its own operands q/k/v may also come as float
partial sums (``ops.linear_summed_later``): up to 16 rows rows CT1 4w 128x2 c48 (4B, 8B; the
32B shape as above), from 17 to 64 rows rows CT2 4w 64x4 c96 (4B, 8B) and 128x2 c80 (32B), else
as above.

65 and 128 rows: the rows of x go as two halves, each to workgroups of its own, with the choices
of 64 rows, for out, down and the q/k/v that a consumer adds; gate/up, the head and a plain q/k/v
go to the library as at 130 rows.
"""
import ctypes
import zlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
VOCAB = 151936
# (hidden, q width, key/value width, feed-forward width)
SIZES = {"4b": (2560, 4096, 1024, 9728), "8b": (4096, 4096, 1024, 12288), "32b": (5120, 8192, 1024, 25600)}
ROWS = (1, 8, 16, 17, 48, 64, 65, 128, 130)

# (kernel, parts, col_tiles, (waves, groups, columns per workgroup)) for few (<= 16) and many
# (17..64) rows; a dict where the many differ among themselves
R = "rows"
EXPECT = {
    ("4b", "qkv"): ((R, 1, 1, (2, 256, 24)), ("library",)),
    ("4b", "out"): ((R, 4, 1, (4, 64, 40)), {17: (R, 4, 1, (4, 64, 40)), 48: (R, 4, 1, (4, 40, 64)),
                                             64: (R, 4, 1, (4, 40, 64))}),
    ("4b", "gate_up"): ((R, 1, 2, (4, 256, 38)), (R, 1, 2, (4, 256, 38))),
    ("4b", "down"): ((R, 4, 1, (4, 64, 40)), (R, 8, 2, (4, 32, 80))),
    ("4b", "head"): ((R, 1, 2, (4, 1277, 119)), (R, 1, 2, (4, 1187, 128))),
    ("8b", "qkv"): ((R, 1, 1, (2, 256, 24)), ("library",)),
    ("8b", "out"): ((R, 4, 1, (4, 64, 64)), (R, 4, 1, (4, 64, 64))),
    ("8b", "gate_up"): (("skinny",), (R, 1, 2, (4, 256, 48))),
    ("8b", "down"): ((R, 4, 1, (4, 64, 64)), (R, 8, 2, (4, 32, 128))),
    ("8b", "head"): ((R, 1, 1, (4, 2533, 60)), {17: (R, 1, 1, (4, 2374, 64)), 48: ("library",), 64: ("library",)}),
    ("32b", "qkv"): ((R, 1, 1, (4, 256, 40)), ("library",)),
    ("32b", "out"): ((R, 4, 2, (4, 64, 80)), (R, 4, 2, (4, 64, 80))),
    ("32b", "gate_up"): ((R, 1, 2, (4, 512, 50)), (R, 1, 2, (4, 512, 50))),
    ("32b", "down"): ((R, 4, 2, (4, 64, 80)), (R, 4, 2, (4, 64, 80))),
    ("32b", "head"): ((R, 1, 2, (4, 1277, 119)), (R, 1, 2, (4, 1187, 128))),
}


# q/k/v for a consumer that adds partial sums: up to 16 rows (the 32B shape is not cut there), 17..64 rows
EXPECT_SUMMED = {"4b": ((R, 2, 1, (4, 128, 48)), (R, 4, 2, (4, 64, 96))),
                 "8b": ((R, 2, 1, (4, 128, 48)), (R, 4, 2, (4, 64, 96))),
                 "32b": (None, (R, 2, 2, (4, 128, 80)))}


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.kernels import check_device, ops as _ops

    check_device()
    return _ops


def shape_of(model: str, product: str):
    hidden, q, kv, inter = SIZES[model]
    return {"qkv": (q + 2 * kv, hidden), "out": (hidden, q), "gate_up": (2 * inter, hidden),
            "down": (hidden, inter), "head": (VOCAB, hidden)}[product]


def launch_shape(rows, n, parts, col_tiles, glu, units=0):
    from pylon_amd.kernels import library

    out = (ctypes.c_int * 3)()
    assert library.load().pylon_gemm_rows_shape(rows, n, parts, col_tiles, glu, 0, units, 0, out) == 0
    return tuple(out)


def chosen(model, product, rows, units):
    """What the plan picks for this case, in the form of EXPECT's entries."""
    from pylon_amd.kernels import plan

    n, k = shape_of(model, product)
    if product in ("out", "down"):
        c = plan.plan_residual(rows, n, k, units=units)
    elif product == "gate_up":
        c = plan.plan_gated(rows, n // 2, k, k)
    else:
        c = plan.plan_projection(rows, n, k)
    if c.kernel != "rows":
        return (c.kernel,)
    glu = product == "gate_up"
    return (c.kernel, c.parts, c.col_tiles, launch_shape(rows, n // 2 if glu else n, c.parts, c.col_tiles, int(glu)))


@pytest.mark.parametrize("product", ["qkv", "out", "gate_up", "down", "head"])
@pytest.mark.parametrize("model", list(SIZES))
def test_a_product_at_its_real_size(ops, model, product):
    from pylon_amd.kernels import library

    n, k = shape_of(model, product)
    gen = torch.Generator(device=DEV).manual_seed(zlib.crc32(f"{model}/{product}".encode()))
    w = (torch.randn((n, k), generator=gen, device=DEV) * 0.02).to(torch.bfloat16)
    x = torch.randn((max(ROWS), k), generator=gen, device=DEV).to(torch.bfloat16)
    want = torch.mm(x.double(), w.double().t())
    if product == "gate_up":
        g, u = want[:, : n // 2], want[:, n // 2:]
        want = g / (1 + torch.exp(-g)) * u
    want = want.cpu().numpy()
    del gen
    few, many = EXPECT[(model, product)]
    units = library.compute_units()
    assert units == 256  # the expectations above are those of an MI355X
    for rows in ROWS:
        if rows <= 64:
            expected = few if rows <= 16 else (many[rows] if isinstance(many, dict) else many)
            assert chosen(model, product, rows, units) == expected, (model, product, rows)
        xr = x[:rows].contiguous()
        if product in ("out", "down"):
            got = ops.linear_for_residual(xr, w, out_dtype=torch.bfloat16)
            if rows <= 128:  # float32 sums, never rounded: whole, or K cut into parts
                assert got.dtype == torch.float32
                if rows > 64:  # two halves of the rows, the choices of 64 rows
                    many64 = many[64] if isinstance(many, dict) else many
                    assert chosen(model, product, rows, units)[:3] == many64[:3], (model, product, rows)
                got = got.sum(0, dtype=torch.float64) if got.dim() == 3 else got
            else:
                assert got.dtype == torch.bfloat16
        elif product == "gate_up":
            got = ops.linear_glu(xr, w, out_dtype=torch.bfloat16)
            assert got.dtype == torch.bfloat16
        elif product == "head":
            got = ops.linear(xr, w, out_dtype=torch.float32)  # logits: float32 at every row count
            assert got.dtype == torch.float32
        else:
            got = ops.linear(xr, w, out_dtype=torch.bfloat16)
            later = ops.linear_summed_later(xr, w, out_dtype=torch.bfloat16)
            from pylon_amd.kernels import plan

            c = plan.plan_summed_later(rows, n, k, units=units)
            if rows <= 128 and c.parts > 1:
                expected = EXPECT_SUMMED[model][0 if rows <= 16 else 1]
                if rows <= 64:
                    assert (c.kernel, c.parts, c.col_tiles, launch_shape(rows, n, c.parts, c.col_tiles, 0)) == \
                        expected, (model, rows)
                else:  # two halves of the rows, the choices of 64 rows
                    assert (c.kernel, c.parts, c.col_tiles) == expected[:3], (model, rows)
                assert later.dtype == torch.float32 and later.shape == (c.parts, rows, n)
                total = later.sum(0, dtype=torch.float64).cpu().numpy()
                assert np.abs(total - want[:rows]).max() <= 2e-6 * np.abs(want[:rows]).max(), (model, rows)
            else:
                assert torch.equal(later, got)
        ref = want[:rows]
        assert got.shape == ref.shape, (model, product, rows, tuple(got.shape))
        scale = np.abs(ref).max()
        # float32 sums: a few ulps of accumulated rounding; bfloat16: one rounding of the result
        # (2^-9), and a second one where the library rounds gate and up before the activation
        # (beyond 128 rows)
        bound = 2e-6 if got.dtype != torch.bfloat16 else (1.2e-2 if product == "gate_up" and rows > 128 else 6e-3)
        error = np.abs(got.double().cpu().numpy() - ref).max()
        assert error <= bound * scale, (model, product, rows, error / scale)
