"""Each kernel alone against a plain float64 reference of the same operation, at sizes
other than the engine's (odd widths, head sizes in steps of 16, vocabularies that are no
power of two), in float32 and in bfloat16."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.kernels import check_device, ops as _ops

    check_device()
    return _ops


def rnd(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def tol(dtype, scale=1.0):
    # float32: a few ulps of accumulated rounding; bfloat16: one rounding of the result
    # (2^-9 relative) plus rounding of inputs that both sides share.
    return (2e-6 if dtype == torch.float32 else 6e-3) * scale


def f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    table = rnd((301, 72), 1, dtype)
    ids = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32)
    out = ops.embed(ids.to(DEV), table.to(DEV), scale=0.5)
    assert out.dtype == torch.float32
    assert np.array_equal(f64(out), f64(table)[ids.numpy()] * 0.5)


def test_sampled_tokens_are_fed_back_on_the_device(ops):
    """argmax / sample leave each row's id in chosen[place[row]]; the embedding takes an id
    -(1 + s) from chosen[s]."""
    vocab = 211
    logits = rnd((3, vocab), 31) * 3
    chosen = torch.full((6,), -7, dtype=torch.int32, device=DEV)
    place = torch.tensor([4, 0, 5], dtype=torch.int32, device=DEV)
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    got = ops.argmax(logits.to(DEV), out=out, chosen=chosen, place=place)
    want = f64(logits).argmax(axis=1).tolist()
    assert got.data_ptr() == out.data_ptr() and got.cpu().tolist() == want
    assert chosen.cpu().tolist() == [want[1], -7, -7, -7, want[0], want[2]]
    temps = torch.tensor([0.0, 0.7, 1.3], device=DEV)
    u = torch.tensor([0.0, 0.3, 0.8], device=DEV)
    plain_draw = ops.sample(logits.to(DEV), temps, torch.ones(3, device=DEV), u).cpu().tolist()
    chosen.fill_(-7)
    drawn = ops.sample(logits.to(DEV), temps, torch.ones(3, device=DEV), u, chosen=chosen, place=place)
    assert drawn.cpu().tolist() == plain_draw
    assert chosen.cpu().tolist() == [plain_draw[1], -7, -7, -7, plain_draw[0], plain_draw[2]]
    table = rnd((vocab, 40), 32)
    ids = torch.tensor([3, -1 - 4, -1 - 0, 9], dtype=torch.int32, device=DEV)
    emb = ops.embed(ids, table.to(DEV), chosen=chosen)
    rows = [3, plain_draw[0], plain_draw[1], 9]
    assert np.array_equal(f64(emb), f64(table)[rows])
    with pytest.raises(Exception):
        ops.argmax(logits.to(DEV), chosen=chosen)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [80, 1000, 2560 + 16])
def test_rmsnorm_and_fused_residual(ops, dtype, dim):
    eps = 3e-5
    x = rnd((7, dim), 2, torch.float32, 2.0)
    delta = rnd((7, dim), 3, dtype)
    w = 1 + 0.3 * rnd((dim,), 4)

    def ref(v):
        return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps) * f64(w)

    got = ops.rmsnorm(x.to(dtype).to(DEV), w.to(DEV), eps, out_dtype=dtype)
    want = ref(f64(x.to(dtype)))
    assert np.abs(f64(got) - want).max() <= tol(dtype, np.abs(want).max())
    # fused: resid += delta (float32), out = norm(resid)
    resid = x.clone().to(DEV)
    got = ops.add_rmsnorm(resid, delta.to(DEV), w.to(DEV), eps, dtype)
    summed = f64(x) + f64(delta)
    assert np.abs(f64(resid) - summed).max() <= 1e-6 * np.abs(summed).max()
    assert np.abs(f64(got) - ref(summed)).max() <= tol(dtype, np.abs(ref(summed)).max())
    # with picked rows the residual stays as it was
    resid = x.clone().to(DEV)
    idx = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    got = ops.add_rmsnorm(resid, delta.to(DEV), w.to(DEV), eps, dtype, row_idx=idx)
    assert torch.equal(resid.cpu(), x)
    assert np.abs(f64(got) - ref(summed)[[6, 0, 3]]).max() <= tol(dtype, np.abs(ref(summed)).max())
    # no delta: plain norm of the residual
    got = ops.add_rmsnorm(resid, None, w.to(DEV), eps, dtype)
    assert np.abs(f64(got) - ref(f64(x))).max() <= tol(dtype, np.abs(ref(f64(x))).max())
    r2 = x.clone().to(DEV)
    ops.residual_add(r2, delta.to(DEV))
    assert np.abs(f64(r2) - summed).max() <= 1e-6 * np.abs(summed).max()


@pytest.mark.parametrize("dim", [80, 2560 + 16, 5120 + 8, 8192])
@pytest.mark.parametrize("delta_dtype", DTYPES)
def test_residual_norm_of_many_rows_has_the_bits_of_few(ops, dim, delta_dtype):
    """From 512 rows on another kernel takes the fused residual norm (two rows a workgroup):
    it forms every row's sums in the order of the kernel for few rows, so a request's values do
    not depend on how many tokens share its step."""
    eps, rows = 1e-6, 515
    x = rnd((rows, dim), 60, torch.float32, 2.0)
    delta = rnd((rows, dim), 61, delta_dtype)
    w = 1 + 0.3 * rnd((dim,), 62)
    summed = f64(x) + f64(delta)
    want = summed / np.sqrt((summed * summed).mean(-1, keepdims=True) + eps) * f64(w)
    for out_dtype in DTYPES:
        many_resid = x.clone().to(DEV)
        many = ops.add_rmsnorm(many_resid, delta.to(DEV), w.to(DEV), eps, out_dtype)
        assert np.abs(f64(many) - want).max() <= tol(out_dtype, np.abs(want).max())
        for lo, hi in ((0, 3), (200, 201), (513, 515)):
            few_resid = x[lo:hi].clone().to(DEV)
            few = ops.add_rmsnorm(few_resid, delta[lo:hi].contiguous().to(DEV), w.to(DEV), eps, out_dtype)
            assert torch.equal(few, many[lo:hi]) and torch.equal(few_resid, many_resid[lo:hi])


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_gate(ops, dtype):
    gu = rnd((5, 2 * 176), 5, dtype, 3.0)
    got = ops.silu_gate(gu.to(DEV))
    g, u = f64(gu)[:, :176], f64(gu)[:, 176:]
    want = g / (1 + np.exp(-g)) * u
    assert np.abs(f64(got) - want).max() <= tol(dtype, np.abs(want).max())
    zero_gate = gu.clone()
    zero_gate[:, :176] = 0
    assert float(ops.silu_gate(zero_gate.to(DEV)).abs().max()) == 0.0


@pytest.mark.parametrize("combo", [
    (torch.float32, torch.float32, torch.float32),
    (torch.bfloat16, torch.bfloat16, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16, torch.float32),
    (torch.bfloat16, torch.float32, torch.bfloat16),
])
@pytest.mark.parametrize("shape", [(1, 96, 80), (5, 301, 176), (67, 130, 1000), (130, 64, 64)])
def test_gemm_tiled(ops, combo, shape):
    a_dt, w_dt, o_dt = combo
    m, n, k = shape
    a, w = rnd((m, k), 6, a_dt), rnd((n, k), 7, w_dt, 0.1)
    got = ops.gemm_tiled(a.to(DEV), w.to(DEV), out_dtype=o_dt)
    want = f64(a) @ f64(w).T
    assert got.dtype == o_dt
    assert np.abs(f64(got) - want).max() <= tol(o_dt, np.abs(want).max())


def test_gemm_rows_do_not_depend_on_the_batch(ops):
    # float32: bit-identical whatever rows share the launch
    a, w = rnd((70, 200), 8), rnd((90, 200), 9)
    whole = ops.gemm_tiled(a.to(DEV), w.to(DEV))
    for lo, hi in ((0, 1), (3, 4), (63, 70), (10, 40)):
        part = ops.gemm_tiled(a[lo:hi].contiguous().to(DEV), w.to(DEV))
        assert torch.equal(part, whole[lo:hi])


@pytest.mark.parametrize("dim", [80, 2560 + 16, 5120 + 8, 9000])
@pytest.mark.parametrize("parts", [1, 2, 3, 4, 8])
def test_residual_norm_adds_partial_sums(ops, dim, parts):
    """A stack of float partial sums of a matrix product (K cut in parts) is added to the
    residual in a fixed order and normed: rows of every width class of the kernel (one that
    fits 256 threads' registers, one that needs 512, one that takes the general loop)."""
    eps, rows = 2e-6, 5
    x = rnd((rows, dim), 12, torch.float32, 2.0)
    stack = rnd((parts, rows, dim), 13, torch.float32)
    w = 1 + 0.3 * rnd((dim,), 14)
    summed = f64(x) + f64(stack).sum(0)
    want = summed / np.sqrt((summed * summed).mean(-1, keepdims=True) + eps) * f64(w)
    for out_dtype in (torch.bfloat16, torch.float32):
        resid = x.clone().to(DEV)
        got = ops.add_rmsnorm(resid, stack.to(DEV), w.to(DEV), eps, out_dtype)
        assert np.abs(f64(resid) - summed).max() <= 1e-6 * np.abs(summed).max()
        assert np.abs(f64(got) - want).max() <= tol(out_dtype, np.abs(want).max())
    # the same bits as adding the parts one after the other in float32
    resid = x.clone().to(DEV)
    ops.add_rmsnorm(resid, stack.to(DEV), w.to(DEV), eps, torch.float32)
    one_by_one = stack[0].clone()
    for p in range(1, parts):
        one_by_one += stack[p]
    assert torch.equal(resid.cpu(), x + one_by_one)
    # picked rows: the residual stays
    resid = x.clone().to(DEV)
    idx = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    got = ops.add_rmsnorm(resid, stack.to(DEV), w.to(DEV), eps, torch.float32, row_idx=idx)
    assert torch.equal(resid.cpu(), x)
    assert np.abs(f64(got) - want[[4, 1]]).max() <= tol(torch.float32, np.abs(want).max())


@pytest.mark.parametrize("shape", [(1, 96, 80), (8, 301, 176), (16, 130, 1000), (17, 64, 64),
                                   (64, 2560 + 8, 512 + 24), (33, 48, 4096), (8, 72, 9728)])
def test_gemm_skinny(ops, shape):
    m, n, k = shape
    a, w = rnd((m, k), 30, torch.bfloat16), rnd((n, k), 31, torch.bfloat16, 0.1)
    want = f64(a) @ f64(w).T
    for out_dtype in (torch.bfloat16, torch.float32):
        got = ops.gemm_skinny(a.to(DEV), w.to(DEV), out_dtype=out_dtype)
        assert got.shape == (m, n) and got.dtype == out_dtype
        assert np.abs(f64(got) - want).max() <= tol(out_dtype, np.abs(want).max())
    for parts in (2, 4, 7):
        got = ops.gemm_skinny(a.to(DEV), w.to(DEV), parts=parts)
        assert got.shape == (parts, m, n) and got.dtype == torch.float32
        assert np.abs(f64(got).sum(0) - want).max() <= tol(torch.float32, np.abs(want).max())
    # the same rows give the same bits whatever other rows share the launch
    full = ops.gemm_skinny(a.to(DEV), w.to(DEV), out_dtype=torch.float32)
    alone = ops.gemm_skinny(a[:1].contiguous().to(DEV), w.to(DEV), out_dtype=torch.float32)
    assert torch.equal(alone, full[:1])
    # gated epilogue over a fused gate/up matrix equals product, then the activation kernel
    if n % 2 == 0:
        both = ops.gemm_skinny(a.to(DEV), w.to(DEV), out_dtype=torch.float32)
        g, u = f64(both)[:, : n // 2], f64(both)[:, n // 2:]
        want_glu = g / (1 + np.exp(-g)) * u
        fused = ops.gemm_skinny(a.to(DEV), w.to(DEV), glu=True)
        assert fused.shape == (m, n // 2)
        assert np.abs(f64(fused) - want_glu).max() <= tol(torch.bfloat16, np.abs(want_glu).max())
        # through the dispatcher, whichever kernel it picks for the shape: one rounding
        via = ops.linear_glu(a.to(DEV), w.to(DEV), out_dtype=torch.bfloat16)
        assert np.abs(f64(via) - want_glu).max() <= tol(torch.bfloat16, np.abs(want_glu).max())
    # through the dispatcher: float32 sums, never rounded, at every row count; refused beyond 64 rows
    via = ops.linear(a.to(DEV), w.to(DEV), out_dtype=torch.float32)
    assert via.dtype == torch.float32
    assert np.abs(f64(via) - want).max() <= tol(torch.float32, np.abs(want).max())
    from pylon_amd.kernels import KernelError
    with pytest.raises(KernelError, match="at most 64 rows"):
        ops.gemm_skinny(torch.zeros((65, 64), dtype=torch.bfloat16, device=DEV), w[:, :64].contiguous().to(DEV))


def test_gemm_rows_at_random_shapes(ops):
    """Ninety seeded draws of every argument (rows 1 to 128, beyond 64 as two halves with
    workgroups of their own; 1 to 700 columns, depths that are multiples of 8 up to 1,496,
    parts beyond the number of chunks, both widths and wave counts, the gated form) against a
    float64 product; and with any number of columns per workgroup, down to one, the bits of
    the kernel's own choice."""
    rng = np.random.default_rng(2024)
    for case in range(90):
        m = int(rng.integers(1, 65)) if case < 60 else int(rng.integers(65, 129))
        k = 8 * int(rng.integers(1, 188))
        glu = bool(rng.integers(0, 2))
        n = int(rng.integers(1, 351)) * (2 if glu else 1) if glu else int(rng.integers(1, 701))
        parts = 1 if glu else int(rng.choice([1, 1, 2, 3, 5, 16]))
        col_tiles, waves = int(rng.choice([1, 2])), int(rng.choice([0, 2, 4]))
        a, w = rnd((m, k), 100 + case, torch.bfloat16), rnd((n, k), 200 + case, torch.bfloat16, 0.1)
        want = f64(a) @ f64(w).T
        if glu:
            g, u = want[:, : n // 2], want[:, n // 2:]
            want = g / (1 + np.exp(-g)) * u
        got = ops.gemm_rows(a.to(DEV), w.to(DEV), out_dtype=torch.float32, parts=parts, col_tiles=col_tiles,
                            glu=glu, waves=waves)
        cols = int(rng.integers(1, 2 * (16 if glu else 16 * col_tiles) + 1))  # what two waves hold at most
        shared = ops.gemm_rows(a.to(DEV), w.to(DEV), out_dtype=torch.float32, parts=parts, col_tiles=col_tiles,
                               glu=glu, waves=waves, cols=cols)
        assert torch.equal(shared, got), (case, m, n, k, parts, col_tiles, glu, waves, cols)
        got = f64(got).sum(0) if parts > 1 else f64(got)
        assert got.shape == want.shape, (case, m, n, k)
        assert np.abs(got - want).max() <= tol(torch.float32, max(np.abs(want).max(), 1e-3)), \
            (case, m, n, k, parts, col_tiles, glu, waves)


@pytest.mark.parametrize("shape", [(17, 100, 200), (64, 2560 + 8, 512 + 24), (33, 61, 136), (50, 333, 1000),
                                   (64, 129, 128), (48, 64, 8), (20, 72, 9728), (1, 77, 264), (16, 300, 392)])
def test_gemm_rows(ops, shape):
    """The product for 17 to 64 rows (x shared through LDS, w streamed, three chunks in
    flight): every size class (rows in 1 to 4 tiles, columns and K that end inside a tile or
    a chunk, K shorter than a chunk), K cut into parts, both workgroup widths."""
    m, n, k = shape
    a, w = rnd((m, k), 32, torch.bfloat16), rnd((n, k), 33, torch.bfloat16, 0.1)
    want = f64(a) @ f64(w).T
    ref = None
    for col_tiles in (1, 2):
        for out_dtype in (torch.bfloat16, torch.float32):
            got = ops.gemm_rows(a.to(DEV), w.to(DEV), out_dtype=out_dtype, col_tiles=col_tiles)
            assert got.shape == (m, n) and got.dtype == out_dtype
            assert np.abs(f64(got) - want).max() <= tol(out_dtype, np.abs(want).max())
        # the two widths add in the same order
        ref = got if ref is None else ref
        assert torch.equal(ref, got)
        for parts in (2, 3, 8, 16):
            got = ops.gemm_rows(a.to(DEV), w.to(DEV), parts=parts, col_tiles=col_tiles)
            assert got.shape == (parts, m, n) and got.dtype == torch.float32
            assert np.abs(f64(got).sum(0) - want).max() <= tol(torch.float32, np.abs(want).max())
    # the same rows give the same bits whatever other rows share the launch
    full = ops.gemm_rows(a.to(DEV), w.to(DEV), parts=4)
    alone = ops.gemm_rows(a[m // 2: m // 2 + 1].contiguous().to(DEV), w.to(DEV), parts=4)
    assert torch.equal(alone[:, 0], full[:, m // 2])
    with pytest.raises(Exception, match="at most 128 rows"):
        ops.gemm_rows(rnd((129, k), 34, torch.bfloat16).to(DEV), w.to(DEV))
    # beyond 64 rows the rows go as two halves: the same bits for a row as in a launch of its own
    tall = torch.cat([a, rnd((100 - m, k), 37, torch.bfloat16)]) if m < 100 else a
    both = ops.gemm_rows(tall.to(DEV), w.to(DEV), parts=4)
    assert both.shape == (4, tall.shape[0], n)
    assert torch.equal(both[:, : m], full) and torch.equal(
        both[:, 99], ops.gemm_rows(tall[99:100].contiguous().to(DEV), w.to(DEV), parts=4)[:, 0])
    # rows of x and w that are slices of wider tensors (strides beyond K)
    wide_x = rnd((m, k + 24), 35, torch.bfloat16).to(DEV)
    wide_w = rnd((n, k + 40), 36, torch.bfloat16, 0.1).to(DEV)
    sliced = ops.gemm_rows(wide_x[:, 8: 8 + k], wide_w[:, 16: 16 + k], out_dtype=torch.float32)
    want_sliced = f64(wide_x[:, 8: 8 + k]) @ f64(wide_w[:, 16: 16 + k]).T
    assert np.abs(f64(sliced) - want_sliced).max() <= tol(torch.float32, np.abs(want_sliced).max())
    # gated epilogue over a fused gate/up matrix equals the product, then the activation
    if n % 2 == 0:
        g, u = want[:, : n // 2], want[:, n // 2:]
        want_glu = g / (1 + np.exp(-g)) * u
        for out_dtype in (torch.bfloat16, torch.float32):
            fused = ops.gemm_rows(a.to(DEV), w.to(DEV), out_dtype=out_dtype, glu=True)
            assert fused.shape == (m, n // 2) and fused.dtype == out_dtype
            assert np.abs(f64(fused) - want_glu).max() <= tol(out_dtype, np.abs(want_glu).max())
        with pytest.raises(Exception, match="whole of K"):
            ops.gemm_rows(a.to(DEV), w.to(DEV), parts=2, glu=True)


def plain_rope(x, pos, inv_freq, rot):
    # x: [..., d]; rotate the first `rot` elements, pairing i with i + rot/2
    ang = (np.float32(pos) * inv_freq.astype(np.float32)).astype(np.float64)
    c, s = np.cos(ang), np.sin(ang)
    out = x.copy()
    a, b = x[..., : rot // 2], x[..., rot // 2: rot]
    out[..., : rot // 2] = a * c - b * s
    out[..., rot // 2: rot] = b * c + a * s
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(5, 5, 48, 48), (6, 2, 16, 16), (3, 1, 128, 64), (2, 2, 80, 0)])
def test_qkv_prepare(ops, dtype, geom):
    nh, nkv, hd, rot = geom
    tokens, page, pages, eps = 9, 4, 6, 2e-5
    qkv = rnd((tokens, (nh + 2 * nkv) * hd), 10, dtype)
    qw, kw = 1 + 0.2 * rnd((hd,), 11), 1 + 0.2 * rnd((hd,), 12)
    inv_freq = (1.0 / (1000.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))) if rot else None
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 1000, 5], dtype=torch.int32)
    slots = torch.tensor([4, 5, 6, 7, 0, 1, 23, 12, -1], dtype=torch.int32)
    kc = torch.zeros((pages, page, nkv, hd), dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    q = torch.empty((tokens, nh, hd), dtype=dtype, device=DEV)
    ops.qkv_prepare(qkv.to(DEV), q, kc, vc, n_heads=nh, n_kv_heads=nkv, head_dim=hd,
                    q_weight=qw.to(DEV), k_weight=kw.to(DEV), eps=eps,
                    inv_freq=inv_freq.to(DEV) if rot else None, rot_dim=rot,
                    positions=positions.to(DEV), slot_map=slots.to(DEV), store_kv=True)
    raw = f64(qkv).reshape(tokens, nh + 2 * nkv, hd)

    def norm(v, w):
        return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps) * f64(w)

    kflat, vflat = f64(kc).reshape(pages * page, nkv, hd), f64(vc).reshape(pages * page, nkv, hd)
    for t in range(tokens):
        qn, kn = norm(raw[t, :nh], qw), norm(raw[t, nh:nh + nkv], kw)
        if rot:
            qn = plain_rope(qn, int(positions[t]), inv_freq.numpy(), rot)
            kn = plain_rope(kn, int(positions[t]), inv_freq.numpy(), rot)
        assert np.abs(f64(q)[t] - qn).max() <= tol(dtype, np.abs(qn).max())
        if slots[t] >= 0:
            assert np.abs(kflat[slots[t]] - kn).max() <= tol(dtype, np.abs(kn).max())
            assert np.array_equal(vflat[slots[t]], raw[t, nh + nkv:])  # v: neither normed nor rotated
    untouched = sorted(set(range(pages * page)) - {int(s) for s in slots if s >= 0})
    assert np.abs(kflat[untouched]).max() == 0 and np.abs(vflat[untouched]).max() == 0
    # without norm weights and without storing: q only, rotated only
    q2 = torch.empty_like(q)
    ops.qkv_prepare(qkv[:, : nh * hd].contiguous().to(DEV), q2, None, None, n_heads=nh, n_kv_heads=nkv,
                    head_dim=hd, q_weight=None, k_weight=None, eps=eps,
                    inv_freq=inv_freq.to(DEV) if rot else None, rot_dim=rot,
                    positions=positions.to(DEV), slot_map=None, store_kv=False)
    for t in range(tokens):
        want = plain_rope(raw[t, :nh], int(positions[t]), inv_freq.numpy(), rot) if rot else raw[t, :nh]
        assert np.abs(f64(q2)[t] - want).max() <= tol(dtype, np.abs(want).max())


def plain_attention(q, keys, values, scale, window):
    """q: [heads, d] at the last position of keys [kv, n, d]."""
    heads = q.shape[0]
    group = heads // keys.shape[0]
    n = keys.shape[1]
    lo = max(0, n - window) if window else 0
    out = np.zeros_like(q)
    for h in range(heads):
        k, v = keys[h // group, lo:], values[h // group, lo:]
        s = k @ q[h] * scale
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ v
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(4, 2, 16, 16, None), (6, 1, 32, 32, None), (5, 5, 48, 16, 70),
                                  (8, 2, 128, 64, None), (2, 1, 256, 16, 33)])
def test_paged_attention(ops, dtype, geom):
    nh, nkv, hd, page, window = geom
    lengths = [1, 65, 130, 2 * page, 2 * page + 1]  # tokens already cached per request (incl. the queries)
    n_pages = sum(-(-n // page) for n in lengths) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(13)).tolist()
    width = max(-(-n // page) for n in lengths)
    table = torch.zeros((len(lengths), width), dtype=torch.int32)
    kc = rnd((n_pages, page, nkv, hd), 14, dtype)
    vc = rnd((n_pages, page, nkv, hd), 15, dtype)
    cursor = 0
    for r, n in enumerate(lengths):
        for i in range(-(-n // page)):
            table[r, i] = perm[cursor]
            cursor += 1
    # queries: the last min(3, n) positions of every request, packed
    tok_row, positions = [], []
    for r, n in enumerate(lengths):
        for p in range(max(0, n - 3), n):
            tok_row.append(r)
            positions.append(p)
    q = rnd((len(tok_row), nh, hd), 16, dtype)
    scale = 1 / math.sqrt(hd)
    got = ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV),
                              torch.tensor(tok_row, dtype=torch.int32, device=DEV),
                              torch.tensor(positions, dtype=torch.int32, device=DEV),
                              page_size=page, window=window, scale=scale)
    kf, vf = f64(kc), f64(vc)
    for i, (r, p) in enumerate(zip(tok_row, positions)):
        idx = [(int(table[r, j // page]), j % page) for j in range(p + 1)]
        keys = np.stack([kf[a, b] for a, b in idx], axis=1)  # [kv, n, d]
        vals = np.stack([vf[a, b] for a, b in idx], axis=1)
        want = plain_attention(f64(q)[i], keys, vals, scale, window)
        assert np.abs(f64(got)[i] - want).max() <= tol(dtype, max(1.0, np.abs(want).max())), (i, r, p)


@pytest.mark.parametrize("geom", [(8, 2, 128, 64, None), (4, 4, 64, 16, None), (16, 1, 256, 32, 100),
                                  (6, 2, 128, 256, None), (1, 1, 64, 16, 7)])
@pytest.mark.parametrize("n_splits,n_cuts", [(1, 1), (2, 1), (4, 1), (8, 1), (1, 2), (4, 3), (8, 8), (2, 64)])
def test_attention_decode(ops, geom, n_splits, n_cuts):
    """Keys shared between the waves of a workgroup (n_splits) and, before that, between
    workgroups (n_cuts): also with more shares than a short request has keys."""
    nh, nkv, hd, page, window = geom
    dtype = torch.bfloat16
    lengths = [1, 15, 16, 17, 65, 300, 2 * page + 1, 700, 70 * page + 3]  # the last: a table of over 64 pages
    n_pages = sum(-(-n // page) for n in lengths) + 2
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(40)).tolist()
    width = max(-(-n // page) for n in lengths)
    table = torch.zeros((len(lengths), width), dtype=torch.int32)
    cursor = 0
    for r, n in enumerate(lengths):
        for i in range(-(-n // page)):
            table[r, i] = perm[cursor]
            cursor += 1
    kc = rnd((n_pages, page, nkv, hd), 41, dtype)
    vc = rnd((n_pages, page, nkv, hd), 42, dtype)
    # poison what no request holds and the slots past each request's end
    held = set()
    for r, n in enumerate(lengths):
        for j in range(n):
            held.add((int(table[r, j // page]), j % page))
    for pg in range(n_pages):
        for off in range(page):
            if (pg, off) not in held:
                kc[pg, off] = float("nan")
                vc[pg, off] = float("nan")
    rows = list(range(len(lengths)))[::-1]  # tokens in another order than the rows
    positions = [lengths[r] - 1 for r in rows]
    q = rnd((len(rows), nh, hd), 43, dtype)
    scale = 1 / math.sqrt(hd)
    args = (q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV),
            torch.tensor(rows, dtype=torch.int32, device=DEV),
            torch.tensor(positions, dtype=torch.int32, device=DEV))
    got = ops.attention_decode(*args, page_size=page, window=window, scale=scale, n_splits=n_splits,
                               n_cuts=n_cuts)
    assert not torch.isnan(got.float()).any()
    kf, vf = f64(kc), f64(vc)
    for i, (r, p) in enumerate(zip(rows, positions)):
        idx = [(int(table[r, j // page]), j % page) for j in range(p + 1)]
        keys = np.stack([kf[a, b] for a, b in idx], axis=1)
        vals = np.stack([vf[a, b] for a, b in idx], axis=1)
        want = plain_attention(f64(q)[i], keys, vals, scale, window)
        err = np.abs(f64(got)[i] - want).max()
        assert err <= tol(dtype, max(1.0, np.abs(want).max())), (i, r, p, err)
    # the general kernel agrees to rounding
    ref = ops.paged_attention(*args, page_size=page, window=window, scale=scale)
    assert float((got.float() - ref.float()).abs().max()) <= 2e-2
    # without row ids token t uses row t of the table
    permuted = table[rows].contiguous()
    same = ops.attention_decode(args[0], args[1], args[2], permuted.to(DEV), None, args[5],
                                page_size=page, window=window, scale=scale, n_splits=n_splits, n_cuts=n_cuts)
    assert torch.equal(same, got)


def test_attention_decode_for_a_large_batch(ops):
    """Three hundred single-token rows in one launch agree with the general kernel."""
    nh, nkv, hd, page, tokens = 8, 2, 64, 16, 300
    gen = torch.Generator().manual_seed(77)
    lengths = torch.randint(1, 200, (tokens,), generator=gen)
    width = int(-(-lengths.max() // page))
    table = torch.randperm(tokens * width, generator=gen).to(torch.int32).reshape(tokens, width)
    kc = rnd((tokens * width, page, nkv, hd), 78, torch.bfloat16).to(DEV)
    vc = rnd((tokens * width, page, nkv, hd), 79, torch.bfloat16).to(DEV)
    q = rnd((tokens, nh, hd), 80, torch.bfloat16).to(DEV)
    pos = (lengths - 1).to(torch.int32).to(DEV)
    rows = torch.arange(tokens, dtype=torch.int32, device=DEV)
    want = ops.paged_attention(q, kc, vc, table.to(DEV), rows, pos, page_size=page, window=None, scale=0.125)
    splits = ops.decode_splits(tokens, nkv, int(lengths.max()))
    got = ops.attention_decode(q, kc, vc, table.to(DEV), None, pos, page_size=page, window=None, scale=0.125,
                               n_splits=splits)
    assert np.abs(f64(got) - f64(want)).max() <= tol(torch.bfloat16, 1.0)


@pytest.mark.parametrize("geom", [(8, 2, 128, 64, None), (4, 4, 64, 16, None), (12, 2, 128, 32, 100),
                                  (5, 1, 256, 16, None), (3, 3, 64, 256, 37), (16, 1, 128, 64, None),
                                  (8, 4, 128, 48, None), (6, 2, 64, 80, 90), (8, 2, 128, 64, 90),
                                  (6, 3, 128, 128, 200), (5, 5, 128, 256, None)])
@pytest.mark.parametrize("rows", [64, 128])
def test_attention_prefill(ops, geom, rows):
    """Portions of several requests at once: starting inside a page, a one-token portion, a
    portion with earlier context; pages in scrambled order, everything unheld poisoned."""
    nh, nkv, hd, page, window = geom
    dtype = torch.bfloat16
    group = nh // nkv
    # (tokens cached before, tokens of this portion)
    portions = [(0, 70), (33, 1), (100, 45), (0, 3), (2 * page - 1, 130), (5, 64)]
    lengths = [a + b for a, b in portions]
    n_pages = sum(-(-n // page) for n in lengths) + 2
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(50)).tolist()
    width = max(-(-n // page) for n in lengths)
    table = torch.zeros((len(lengths), width), dtype=torch.int32)
    cursor = 0
    for r, n in enumerate(lengths):
        for i in range(-(-n // page)):
            table[r, i] = perm[cursor]
            cursor += 1
    kc = rnd((n_pages, page, nkv, hd), 51, dtype)
    vc = rnd((n_pages, page, nkv, hd), 52, dtype)
    held = {(int(table[r, j // page]), j % page) for r, n in enumerate(lengths) for j in range(n)}
    for pg in range(n_pages):
        for off in range(page):
            if (pg, off) not in held:
                kc[pg, off] = float("nan")
                vc[pg, off] = float("nan")
    tok_row, positions, tiles = [], [], []
    per_tile = rows // group
    for r, (before, count) in enumerate(portions):
        for lo in range(0, count, per_tile):
            tiles.append((len(tok_row) + lo, min(per_tile, count - lo), r, before + lo))
        tok_row += [r] * count
        positions += list(range(before, before + count))
    tiles = tiles[::-1]  # any order
    q = rnd((len(tok_row), nh, hd), 53, dtype)
    scale = 1 / math.sqrt(hd)
    got = ops.attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV),
                                torch.tensor(tiles, dtype=torch.int32, device=DEV),
                                page_size=page, window=window, scale=scale, rows=rows)
    assert not torch.isnan(got.float()).any()
    kf, vf = f64(kc), f64(vc)
    worst = 0.0
    for i, (r, p) in enumerate(zip(tok_row, positions)):
        idx = [(int(table[r, j // page]), j % page) for j in range(p + 1)]
        keys = np.stack([kf[a, b] for a, b in idx], axis=1)
        vals = np.stack([vf[a, b] for a, b in idx], axis=1)
        want = plain_attention(f64(q)[i], keys, vals, scale, window)
        err = np.abs(f64(got)[i] - want).max()
        # probabilities are rounded to bfloat16 before they weigh the values
        assert err <= 2 * tol(dtype, max(1.0, np.abs(want).max())), (i, r, p, err)
        worst = max(worst, err)
    ref = ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV),
                              torch.tensor(tok_row, dtype=torch.int32, device=DEV),
                              torch.tensor(positions, dtype=torch.int32, device=DEV),
                              page_size=page, window=window, scale=scale)
    assert float((got.float() - ref.float()).abs().max()) <= 3e-2


@pytest.mark.parametrize("kernel", ["general_f32", "general_bf16", "decode", "prefill", "prefill_direct"])
def test_attention_finds_one_far_key_among_hundreds(ops, kernel):
    # Random keys would hide a key that is skipped; here one far key matches the query
    # exactly and strongly, so the output must be (almost) that key's value.
    dtype = torch.float32 if kernel == "general_f32" else torch.bfloat16
    nh, nkv, hd, page = 2, 1, 64, 16
    if kernel == "prefill_direct":  # the prompt kernel that loads whole blocks of a page into LDS
        hd, page = 128, 64
    n = 777
    for far in (0, 15, 16, 63, 64, 400, 776 - 64, 767, 768, 775, 776):
        kc = (rnd((50, page, nkv, hd), 17) * 0.01).to(dtype)
        vc = rnd((50, page, nkv, hd), 18).to(dtype)
        table = torch.arange(49, -1, -1, dtype=torch.int32).reshape(1, 50)
        q = rnd((1, nh, hd), 19).to(dtype)
        page_id, off = int(table[0, far // page]), far % page
        kc[page_id, off, 0] = (q[0, 0].float() * 4.0).to(dtype)
        row = torch.zeros(1, dtype=torch.int32, device=DEV)
        pos = torch.tensor([n - 1], dtype=torch.int32, device=DEV)
        args = (q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV))
        if kernel == "decode":
            got = ops.attention_decode(*args, row, pos, page_size=page, window=None, scale=1.0, n_splits=8)
        elif kernel.startswith("prefill"):
            tiles = torch.tensor([[0, 1, 0, n - 1]], dtype=torch.int32, device=DEV)
            got = ops.attention_prefill(*args, tiles, page_size=page, window=None, scale=1.0)
        else:
            got = ops.paged_attention(*args, row, pos, page_size=page, window=None, scale=1.0)
        assert torch.allclose(got[0, 0].float().cpu(), vc[page_id, off, 0].float(), atol=2e-2), (kernel, far)


@pytest.mark.parametrize("kernel", ["general", "decode", "prefill", "prefill_direct"])
def test_attention_window_edge_fast_kernels(ops, kernel):
    # the key at distance `window` must be invisible, the one at distance window-1 visible
    nh, nkv, hd, page, window = 1, 1, 64, 16, 37
    if kernel == "prefill_direct":
        hd, page = 128, 64
    dtype = torch.bfloat16
    kc = torch.zeros((8, page, nkv, hd), dtype=dtype)
    vc = rnd((8, page, nkv, hd), 20, dtype)
    table = torch.arange(8, dtype=torch.int32).reshape(1, 8)
    q = torch.ones((1, nh, hd), dtype=dtype)
    pos = 100
    row = torch.zeros(1, dtype=torch.int32, device=DEV)
    p = torch.tensor([pos], dtype=torch.int32, device=DEV)
    for key, visible in ((pos - window, False), (pos - window + 1, True)):
        k2 = kc.clone()
        k2[key // page, key % page, 0] = 1.0  # a key that dominates: score 64 against 0
        args = (q.to(DEV), k2.to(DEV), vc.to(DEV), table.to(DEV))
        if kernel == "decode":
            got = ops.attention_decode(*args, row, p, page_size=page, window=window, scale=1.0, n_splits=2)
        elif kernel.startswith("prefill"):
            tiles = torch.tensor([[0, 1, 0, pos]], dtype=torch.int32, device=DEV)
            got = ops.attention_prefill(*args, tiles, page_size=page, window=window, scale=1.0)
        else:
            got = ops.paged_attention(*args, row, p, page_size=page, window=window, scale=1.0)
        hit = torch.allclose(got[0, 0].float().cpu(), vc[key // page, key % page, 0].float(), atol=2e-2)
        assert hit == visible, (kernel, key)


def test_attention_window_edge(ops):
    # the key at distance `window` must be invisible, the one at distance window-1 visible
    nh, nkv, hd, page, window = 1, 1, 16, 16, 37
    kc = torch.zeros((8, page, nkv, hd))
    vc = rnd((8, page, nkv, hd), 20)
    table = torch.arange(8, dtype=torch.int32).reshape(1, 8)
    q = torch.ones((1, nh, hd))
    pos = 100
    for key, visible in ((pos - window, False), (pos - window + 1, True)):
        k2 = kc.clone()
        k2[key // page, key % page, 0] = 8.0  # a key that would dominate
        got = ops.paged_attention(q.to(DEV), k2.to(DEV), vc.to(DEV), table.to(DEV),
                                  torch.zeros(1, dtype=torch.int32, device=DEV),
                                  torch.tensor([pos], dtype=torch.int32, device=DEV),
                                  page_size=page, window=window, scale=1.0)
        hit = torch.allclose(got[0, 0].cpu(), vc[key // page, key % page, 0], atol=1e-3)
        assert hit == visible, key


def test_sampling_kernels(ops):
    from tests.plain import qwen3 as plain

    vocab = 1237
    logits = rnd((6, vocab), 21, scale=3.0)
    logits[2, 55] = logits[2, 900] = logits[2].max() + 1  # a tie: the lowest index wins
    dev = logits.to(DEV)
    assert ops.argmax(dev).cpu().tolist() == [int(np.argmax(f64(logits)[r])) for r in range(6)]
    assert ops.argmax(dev).cpu().tolist()[2] == 55
    temps = torch.tensor([0.0, 0.7, 1.0, 1.3, 0.5, 2.0])
    tops = torch.tensor([1.0, 1.0, 0.9, 0.5, 0.05, 0.95])
    for trial in range(12):
        u = torch.rand(6, generator=torch.Generator().manual_seed(100 + trial))
        got = ops.sample(dev, temps.to(DEV), tops.to(DEV), u.to(DEV)).cpu().tolist()
        for r in range(6):
            p = plain.sampling_distribution(f64(logits)[r], float(temps[r]), float(tops[r])) if temps[r] > 0 else None
            want = plain.sample_with_uniform(f64(logits)[r], float(temps[r]), float(tops[r]), float(u[r]))
            if got[r] != want:
                # float32 sums may land on the other side of a boundary of the cumulative
                # distribution; then the draw must be an adjacent kept token and u must
                # lie within rounding of that boundary.
                cdf = np.cumsum(p)
                assert p[got[r]] > 0 and abs(cdf[min(got[r], want)] - float(u[r])) < 1e-5, (trial, r)
    # top-p keeps exactly the tokens the plain rule keeps: with u just below 1 the draw is
    # the last kept token in vocabulary order
    almost_one = torch.full((6,), 1.0 - 2 ** -24)
    got = ops.sample(dev, temps.to(DEV), tops.to(DEV), almost_one.to(DEV)).cpu().tolist()
    for r in range(1, 6):
        p = plain.sampling_distribution(f64(logits)[r], float(temps[r]), float(tops[r]))
        assert got[r] == int(np.nonzero(p)[0][-1]), r
    # empirical frequencies match softmax on a small distribution
    small = torch.log(torch.tensor([[0.5, 0.25, 0.125, 0.125]])).repeat(4000, 1).to(DEV)
    us = torch.rand(4000, generator=torch.Generator().manual_seed(3)).to(DEV)
    draws = ops.sample(small, torch.ones(4000, device=DEV), torch.ones(4000, device=DEV), us).cpu().numpy()
    freq = np.bincount(draws, minlength=4) / 4000
    assert np.abs(freq - [0.5, 0.25, 0.125, 0.125]).max() < 0.03


def _check_draws(ops, logits, temps, tops, us, plain):
    """Every draw is the plain rule's, or an adjacent kept token with u on that boundary of
    the cumulative distribution."""
    got = ops.sample(logits.to(DEV), temps.to(DEV), tops.to(DEV), us.to(DEV)).cpu().tolist()
    again = ops.sample(logits.to(DEV), temps.to(DEV), tops.to(DEV), us.to(DEV)).cpu().tolist()
    assert got == again  # integer masses: the same on every run
    for r in range(logits.shape[0]):
        row = f64(logits)[r]
        want = plain.sample_with_uniform(row, float(temps[r]), float(tops[r]), float(us[r]))
        if got[r] != want:
            p = plain.sampling_distribution(row, float(temps[r]), float(tops[r]))
            cdf = np.cumsum(p)
            assert p[got[r]] > 0 and abs(cdf[min(got[r], want)] - float(us[r])) < 1e-5, (r, got[r], want)
    return got


def test_sampling_at_a_full_vocabulary_and_odd_layouts(ops):
    from tests.plain import qwen3 as plain

    # a real vocabulary; rows that start at addresses that are no multiple of 16 bytes
    vocab = 151936
    base = rnd((5, vocab + 3), 41, scale=2.5)
    logits = base[:, 1: 1 + vocab]  # row stride vocab + 3, first element off by one float
    assert logits.stride(0) == vocab + 3
    dev_base = base.to(DEV)
    dev = dev_base[:, 1: 1 + vocab]
    temps = torch.tensor([1.0, 0.6, 0.2, 1.5, 0.9])
    tops = torch.tensor([0.95, 0.5, 0.95, 1.0, 0.999])
    assert ops.argmax(dev).cpu().tolist() == f64(logits).argmax(axis=1).tolist()
    for trial in range(4):
        us = torch.rand(5, generator=torch.Generator().manual_seed(7 + trial))
        got = ops.sample(dev, temps.to(DEV), tops.to(DEV), us.to(DEV)).cpu().tolist()
        for r in range(5):
            row = f64(logits)[r]
            want = plain.sample_with_uniform(row, float(temps[r]), float(tops[r]), float(us[r]))
            if got[r] != want:
                p = plain.sampling_distribution(row, float(temps[r]), float(tops[r]))
                cdf = np.cumsum(p)
                assert p[got[r]] > 0 and abs(cdf[min(got[r], want)] - float(us[r])) < 1e-5, (trial, r)
    # the kept set: u just below 1 draws the last kept token in vocabulary order
    almost_one = torch.full((5,), 1.0 - 2 ** -24)
    got = ops.sample(dev, temps.to(DEV), tops.to(DEV), almost_one.to(DEV)).cpu().tolist()
    for r in range(5):
        p = plain.sampling_distribution(f64(logits)[r], float(temps[r]), float(tops[r]))
        kept = np.nonzero(p > 2.0 ** -40)[0]
        assert got[r] == int(kept[-1]), r
    # u = 0 draws the first kept token
    got = ops.sample(dev, temps.to(DEV), tops.to(DEV), torch.zeros(5, device=DEV)).cpu().tolist()
    for r in range(5):
        p = plain.sampling_distribution(f64(logits)[r], float(temps[r]), float(tops[r]))
        assert got[r] == int(np.nonzero(p > 2.0 ** -40)[0][0]), r


def test_sampling_with_thousands_of_equal_logits_at_the_boundary(ops):
    """More tokens in the top-p boundary's bin than the kernel gathers in LDS, most of them
    equal: the kept set is the plain rule's, made whole where that rule cuts into a tie."""
    from tests.plain import qwen3 as plain

    vocab = 20000
    gen = torch.Generator().manual_seed(5)
    logits = torch.full((3, vocab), -4.0)
    logits[:, :50] = 2.0 + torch.rand((3, 50), generator=gen)  # a head that holds ~60 % of the mass
    logits[:, 50:9000] = 0.0                                       # 8950 equal tokens
    logits[1, 50:9000] += torch.rand(8950, generator=gen) * 1e-3   # ... or nearly equal
    logits[2, 9000:] = -30.0
    temps = torch.ones(3)
    for top_p in (0.7, 0.95):
        tops = torch.full((3,), top_p)
        dev = logits.to(DEV)
        almost_one = torch.full((3,), 1.0 - 2 ** -24)
        last = ops.sample(dev, temps.to(DEV), tops.to(DEV), almost_one.to(DEV)).cpu().tolist()
        first = ops.sample(dev, temps.to(DEV), tops.to(DEV), torch.zeros(3, device=DEV)).cpu().tolist()
        for r in range(3):
            row = f64(logits)[r]
            # The plain rule sorts and cuts wherever the cumulative mass passes top_p, inside a
            # tie too (which of the equal tokens it keeps is an accident of its sort).  The
            # kernel keeps every token at least as large as the smallest one the plain rule
            # keeps: the same set, plus the rest of a tie the plain rule cut into.
            p = plain.sampling_distribution(row, 1.0, top_p)
            smallest_kept = row[p > 0].min()
            mass = np.exp(row - row.max())
            kept = np.nonzero((row >= smallest_kept) & (mass * 2.0 ** 40 >= 1))[0]
            assert first[r] == int(kept[0]) and last[r] == int(kept[-1]), (top_p, r, first[r], last[r])
    us = torch.tensor([0.3, 0.6, 0.9])
    _check_draws(ops, logits[1:2].repeat(3, 1), temps, torch.full((3,), 0.7), us, plain)


def test_sampling_with_logits_that_are_not_numbers_and_small_vocabularies(ops):
    """NaN counts as -inf, for the argmax and for a draw; a row that is -inf throughout gives
    token 0 and one with +inf its first +inf; vocabularies smaller than a wave's group of
    loads, and just beyond what the last scan takes, draw by the plain rule."""
    from tests.plain import qwen3 as plain

    nan, inf = float("nan"), float("inf")
    for vocab in (3, 64, 1024, 1025, 5000):
        gen = torch.Generator().manual_seed(vocab)
        logits = 2.0 * torch.randn((6, vocab), generator=gen)
        logits[0, ::2] = nan
        logits[1, 1::3] = -inf
        logits[2, :] = -inf
        logits[3, :] = nan
        logits[4, vocab // 2] = inf
        logits[4, vocab - 1] = inf
        cleaned = torch.where(torch.isnan(logits), torch.full_like(logits, -inf), logits)
        want_top = [int(np.argmax(f64(cleaned)[r])) for r in range(6)]
        want_top[2] = want_top[3] = 0
        want_top[4] = vocab // 2
        dev = logits.to(DEV)
        assert ops.argmax(dev).cpu().tolist() == want_top, vocab
        temps = torch.tensor([0.7, 1.0, 1.0, 0.5, 1.0, 0.0])
        tops = torch.tensor([1.0, 0.8, 0.9, 1.0, 0.95, 0.9])
        for trial in range(4):
            us = torch.rand(6, generator=torch.Generator().manual_seed(trial))
            got = ops.sample(dev, temps.to(DEV), tops.to(DEV), us.to(DEV)).cpu().tolist()
            assert [got[2], got[3], got[4], got[5]] == [0, 0, vocab // 2, want_top[5]], (vocab, trial, got)
            for r in (0, 1):
                row = f64(cleaned)[r]
                want = plain.sample_with_uniform(row, float(temps[r]), float(tops[r]), float(us[r]))
                if got[r] != want:
                    p = plain.sampling_distribution(row, float(temps[r]), float(tops[r]))
                    cdf = np.cumsum(p)
                    assert p[got[r]] > 0 and abs(cdf[min(got[r], want)] - float(us[r])) < 1e-5, (vocab, trial, r)
    # a temperature so low that only the largest logit has mass: the argmax, whatever u
    logits = 2.0 * torch.randn((3, 3000), generator=torch.Generator().manual_seed(1))
    got = ops.sample(logits.to(DEV), torch.full((3,), 1e-3).to(DEV), torch.full((3,), 0.95).to(DEV),
                     torch.tensor([0.0, 0.5, 0.999]).to(DEV)).cpu().tolist()
    assert got == f64(logits).argmax(axis=1).tolist()


def test_sampling_where_most_of_the_row_has_no_mass(ops):
    """Logits as a trained model's: a handful of tokens carry all the mass and whole stretches
    of the row lie too far below to have any, which the passes step over 256 tokens at a time.
    The draws are still the plain rule's, from the first stretch to the last token."""
    from tests.plain import qwen3 as plain

    vocab = 70001
    gen = torch.Generator().manual_seed(11)
    logits = -40.0 - torch.rand((4, vocab), generator=gen)
    for r, places in enumerate(([5, 20000, 70000], [0, 1, 2, 3], [4352, 4353, 35000, 69999], [12345])):
        logits[r, places] = torch.tensor([1.0, 0.5, 0.2, -0.3])[: len(places)]
    # a stretch with a little mass at temperature 1 and none at 0.2 (no two alike: a tie at the
    # top-p boundary is kept whole by the kernel and cut by the plain rule)
    logits[2, 60000:60300] = -6.0 - 2.0 * torch.rand(300, generator=gen)
    for temp, top_p in ((1.0, 1.0), (1.0, 0.9), (0.2, 0.95), (0.2, 1.0), (2.0, 0.5)):
        temps, tops = torch.full((4,), temp), torch.full((4,), top_p)
        for trial in range(6):
            us = torch.rand(4, generator=torch.Generator().manual_seed(50 + trial))
            _check_draws(ops, logits, temps, tops, us, plain)
        # the ends of the kept set
        first = ops.sample(logits.to(DEV), temps.to(DEV), tops.to(DEV), torch.zeros(4, device=DEV)).cpu().tolist()
        last = ops.sample(logits.to(DEV), temps.to(DEV), tops.to(DEV),
                          torch.full((4,), 1.0 - 2 ** -24).to(DEV)).cpu().tolist()
        for r in range(4):
            p = plain.sampling_distribution(f64(logits)[r], temp, top_p)
            kept = np.nonzero(p > 2.0 ** -40)[0]
            assert first[r] == int(kept[0]) and last[r] == int(kept[-1]), (temp, top_p, r, first[r], last[r])


@pytest.mark.parametrize("geom", [(8, 2, 128, True, True), (6, 6, 64, True, False), (5, 1, 256, False, True),
                                  (16, 1, 64, True, True), (3, 3, 128, False, False)])
@pytest.mark.parametrize("store", [True, False])
def test_decode_attention_that_prepares_q_k_v_itself(ops, geom, store):
    """One launch from the raw projection gives the bits of the two launches it replaces:
    the prepared queries' attention output, and the key and value rows in the cache."""
    nh, nkv, hd, normed, rotated = geom
    page, pages, tokens, eps = 16, 40, 7, 3e-6
    width = (nh + (2 * nkv if store else 0)) * hd
    qkv = rnd((tokens, width), 51, torch.bfloat16).to(DEV)
    qw = (1 + 0.2 * rnd((hd,), 52)).to(DEV) if normed else None
    kw = (1 + 0.2 * rnd((hd,), 53)).to(DEV) if normed else None
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))).to(DEV) if rotated else None
    lengths = [1, 17, 64, 65, 200, 16, 333]  # the new token is the last of each
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    perm = torch.randperm(pages * 4, generator=torch.Generator().manual_seed(9)).to(torch.int32)
    table = perm[: tokens * 21].reshape(tokens, 21) % (pages * 4)
    # distinct pages per request so that no two tokens share a slot
    table = torch.arange(tokens * 21, dtype=torch.int32).reshape(tokens, 21)
    total_pages = tokens * 21
    slots = torch.tensor([int(table[t, (n - 1) // page]) * page + (n - 1) % page for t, n in enumerate(lengths)],
                         dtype=torch.int32)
    kc = (rnd((total_pages, page, nkv, hd), 54, torch.bfloat16) * 0.5).to(DEV)
    vc = rnd((total_pages, page, nkv, hd), 55, torch.bfloat16).to(DEV)
    kc2, vc2 = kc.clone(), vc.clone()
    for window in (None, 50):
        for splits, cuts in ((1, 1), (4, 1), (8, 1), (2, 3), (8, 4)):
            q = torch.empty((tokens, nh, hd), dtype=torch.bfloat16, device=DEV)
            ops.qkv_prepare(qkv, q, kc, vc, n_heads=nh, n_kv_heads=nkv, head_dim=hd, q_weight=qw, k_weight=kw,
                            eps=eps, inv_freq=inv_freq, rot_dim=hd if rotated else 0,
                            positions=positions.to(DEV), slot_map=slots.to(DEV), store_kv=store)
            want = ops.attention_decode(q, kc, vc, table.to(DEV), None, positions.to(DEV), page_size=page,
                                        window=window, scale=hd ** -0.5, n_splits=splits, n_cuts=cuts)
            got = ops.attention_decode_fused(
                qkv, kc2, vc2, table.to(DEV), None, positions.to(DEV), n_heads=nh, q_weight=qw, k_weight=kw,
                eps=eps, inv_freq=inv_freq, slot_map=slots.to(DEV) if store else None, page_size=page,
                window=window, scale=hd ** -0.5, n_splits=splits, n_cuts=cuts)
            assert torch.equal(got, want), (window, splits, cuts)
            assert torch.equal(kc2, kc) and torch.equal(vc2, vc)
    # The projection as float partial sums (a product whose K was cut over workgroups): added in
    # order and rounded to bfloat16 once, they give the bits of the projection so rounded.
    for parts in (2, 3, 4, 7):
        stack = rnd((parts, tokens, width), 60 + parts).to(DEV)
        total = stack[0].clone()
        for p in range(1, parts):
            total = total + stack[p]
        rounded = total.to(torch.bfloat16)
        kc3, vc3, kc4, vc4 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
        common = dict(n_heads=nh, q_weight=qw, k_weight=kw, eps=eps, inv_freq=inv_freq,
                      slot_map=slots.to(DEV) if store else None, page_size=page, window=None, scale=hd ** -0.5,
                      n_splits=4, n_cuts=2)
        want = ops.attention_decode_fused(rounded, kc3, vc3, table.to(DEV), None, positions.to(DEV), **common)
        got = ops.attention_decode_fused(stack, kc4, vc4, table.to(DEV), None, positions.to(DEV), **common)
        assert torch.equal(got, want), parts
        assert torch.equal(kc4, kc3) and torch.equal(vc4, vc3), parts


def test_kernels_refuse_what_they_cannot_do(ops):
    from pylon_amd.kernels import KernelError

    q = torch.zeros((1, 2, 24), device=DEV)
    kc = torch.zeros((2, 16, 1, 24), device=DEV)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelError, match="multiple of 16"):
        ops.paged_attention(q, kc, kc, torch.zeros((1, 1), dtype=torch.int32, device=DEV), z, z,
                            page_size=16, window=None, scale=1.0)
    with pytest.raises(KernelError, match="cannot be grouped"):
        ops.paged_attention(torch.zeros((1, 3, 32), device=DEV), torch.zeros((2, 16, 2, 32), device=DEV),
                            torch.zeros((2, 16, 2, 32), device=DEV),
                            torch.zeros((1, 1), dtype=torch.int32, device=DEV), z, z,
                            page_size=16, window=None, scale=1.0)
    with pytest.raises(KernelError, match="no CPU path"):
        ops.rmsnorm(torch.zeros((2, 8)), torch.ones(8), 1e-6)
    with pytest.raises(KernelError, match="float32 and bfloat16"):
        ops.rmsnorm(torch.zeros((2, 8), dtype=torch.float16, device=DEV), torch.ones(8, device=DEV), 1e-6)
    with pytest.raises(KernelError, match="cannot multiply"):
        ops.gemm_tiled(torch.zeros((2, 8), device=DEV), torch.zeros((4, 9), device=DEV))


def test_products_have_one_precision_at_every_row_count(ops):
    """What a row's product is rounded to must not depend on how many rows share the call: the
    logits (float32 result) and the products added to the residual stream are float32 sums
    that were never rounded, from the weight-streaming kernel up to 16 rows and with the
    library taking part beyond; the gated activation works on float32 sums and is rounded
    once.  Rows of different calls then agree to float32 accuracy (the activation: up to rare
    flips by one bfloat16 unit where a sum sits on a rounding boundary)."""
    gen = torch.Generator().manual_seed(5)
    k, inter = 2560, 1280
    x = torch.randn((64, k), generator=gen).to(torch.bfloat16).to(DEV)
    head = (torch.randn((3001, k), generator=gen) * 0.02).to(torch.bfloat16).to(DEV)
    down = (torch.randn((k, 5120), generator=gen) * 0.02).to(torch.bfloat16).to(DEV)
    wide = torch.randn((64, 5120), generator=gen).to(torch.bfloat16).to(DEV)
    gate_up = (torch.randn((2 * inter, k), generator=gen) * 0.02).to(torch.bfloat16).to(DEV)
    ref_head = x[0].double() @ head.double().T
    ref_down = wide[0].double() @ down.double().T
    gu = x[0].double() @ gate_up.double().T
    ref_act = torch.nn.functional.silu(gu[:inter]) * gu[inter:]
    acts = []
    for rows in (1, 16, 17, 33, 64):
        logits = ops.linear(x[:rows].contiguous(), head, out_dtype=torch.float32)
        assert logits.dtype == torch.float32
        assert float((logits[0].double() - ref_head).abs().max()) <= 2e-6 * float(ref_head.abs().max()), rows
        delta = ops.linear_for_residual(wide[:rows].contiguous(), down, out_dtype=torch.bfloat16)
        assert delta.dtype == torch.float32
        total = delta.sum(dim=0) if delta.dim() == 3 else delta
        assert float((total[0].double() - ref_down).abs().max()) <= 2e-6 * float(ref_down.abs().max()), rows
        act = ops.linear_glu(x[:rows].contiguous(), gate_up, out_dtype=torch.bfloat16)
        assert float((act[0].double() - ref_act).abs().max()) <= 2.0 ** -8 * float(ref_act.abs().max()), rows
        acts.append(act[0].float())
    for other in acts[1:]:
        assert float((other != acts[0]).float().mean()) <= 5e-3  # one rounding each: they differ by rare flips only
        assert float((other - acts[0]).abs().max()) <= 2.0 ** -7 * float(acts[0].abs().max())
