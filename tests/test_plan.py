"""The choice of product kernel by shape (pylon_amd/kernels/plan.py): pure functions, checked
here without a GPU for the sizes of every Qwen3 dense model and for the properties the
kernels rely on."""
import pytest

from pylon_amd.kernels import plan

# (hidden, q width, key/value width, feed-forward width) of the published Qwen3 dense sizes
SIZES = {
    "0.6b": (1024, 2048, 1024, 3072),
    "1.7b": (2048, 2048, 1024, 6144),
    "4b": (2560, 4096, 1024, 9728),
    "8b": (4096, 4096, 1024, 12288),
    "14b": (5120, 5120, 1024, 17408),
    "32b": (5120, 8192, 1024, 25600),
}
VOCAB = 151936


@pytest.mark.parametrize("rows", [1, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("name", list(SIZES))
def test_every_choice_is_one_the_kernels_take(name, rows):
    hidden, q, kv, inter = SIZES[name]
    for n, k in ((hidden, q), (hidden, inter)):
        c = plan.plan_residual(rows, n, k)
        assert c.kernel in ("rows", "skinny", "library")
        if c.kernel == "rows":
            groups = -(-n // (64 * c.col_tiles))
            assert c.col_tiles in (1, 2) and 1 <= c.parts <= 16
            assert c.parts == 1 or (c.parts * groups <= plan.UNITS and k // c.parts >= 256)
        if c.kernel == "skinny":
            assert rows <= plan.FEW_ROWS and 1 <= c.parts <= 4
    for n, k in ((q + 2 * kv, hidden), (VOCAB, hidden)):
        c = plan.plan_projection(rows, n, k)
        assert c.parts == 1  # nothing adds partial sums behind these
        assert c.kernel != "skinny" or rows <= plan.FEW_ROWS
    c = plan.plan_gated(rows, inter, hidden, hidden)
    assert c.parts == 1 and (c.kernel != "skinny" or rows <= plan.FEW_ROWS)
    assert c.kernel != "rows" or c.col_tiles == 2  # a wave's gate tile and its up tile


def test_the_benchmark_shape_streams_nearly_everything_through_the_rows_kernel():
    hidden, q, kv, inter = SIZES["4b"]
    for rows in (1, 8, 16, 64):
        assert plan.plan_projection(rows, q + 2 * kv, hidden).kernel == ("rows" if rows <= 16 else "library")
        assert plan.plan_projection(rows, VOCAB, hidden) == plan.Product("rows", 1, 2)
        assert plan.plan_gated(rows, inter, hidden, hidden).kernel == "rows"
        assert plan.plan_residual(rows, hidden, q) == plan.Product("rows", 4, 1)
    assert plan.plan_residual(8, hidden, inter) == plan.Product("rows", 4, 1)
    assert plan.plan_residual(64, hidden, inter) == plan.Product("rows", 8, 2)


def test_rows_of_a_power_of_two_length_and_small_matrices_keep_the_other_kernels():
    hidden, q, kv, inter = SIZES["8b"]
    assert plan.aliased_rows(hidden) and not plan.aliased_rows(2560) and not plan.aliased_rows(2048)
    assert plan.plan_gated(8, inter, hidden, hidden).kernel == "skinny"
    assert plan.plan_gated(64, inter, hidden, hidden).kernel == "rows"
    assert plan.plan_projection(48, q + 2 * kv, hidden).kernel == "library"
    assert plan.plan_projection(8, q + 2 * kv, hidden).kernel == "rows"
    assert plan.plan_projection(8, VOCAB, hidden) == plan.Product("rows", 1, 1)   # 64 columns a workgroup
    assert plan.plan_projection(32, VOCAB, hidden) == plan.Product("rows", 1, 1)
    assert plan.plan_projection(33, VOCAB, hidden).kernel == "library"
    assert plan.plan_gated(8, 3072, 1024, 1024).kernel == "skinny"      # a small matrix
    assert plan.plan_gated(64, 25600, 5120, 5120).kernel == "rows"      # from 17 rows whatever the width
    assert plan.plan_residual(64, 8192, 8192).kernel == "library"       # wide, and rows of a power-of-two length
    assert plan.plan_residual(64, 16384, 4096).kernel == "library"
    assert plan.plan_residual(64, 5120, 8192) == plan.Product("rows", 4, 2)   # not wide
    assert plan.plan_residual(64, 10240, 10240).kernel == "rows"        # wide, rows of another length
    assert plan.plan_residual(8, 16384, 8192).kernel == "skinny"


def test_gate_up_rows_are_kept_apart_in_memory():
    """64 unused elements behind every row of 16-bit elements, none in the 32-bit path; with them
    the rows kernel takes the 8B gate/up (rows of 8 KB) at few rows too."""
    assert plan.gated_row_padding(4096, 2) == 64 and plan.gated_row_padding(2560, 2) == 64
    assert plan.gated_row_padding(4096, 4) == 0  # the 32-bit path's matrices stay as they are
    assert plan.gated_row_padding(96, 2) == 0    # nor is a toy's matrix doubled
    assert plan.plan_gated(8, 12288, 4096, 4096).kernel == "skinny"
    assert plan.plan_gated(8, 12288, 4096, 4096 + 64) == plan.Product("rows", 1, 2)
    assert plan.plan_gated(64, 12288, 4096, 4096 + 64) == plan.Product("rows", 1, 2)


def test_a_gate_up_matrix_beyond_a_descriptor_is_not_given_to_the_rows_kernel():
    assert plan.plan_gated(8, 300_000, 2560, 4096).kernel == "skinny"   # 300,064 rows x 8 KB > 2 GB
    assert plan.plan_gated(64, 300_000, 2560, 4096).kernel == "library"


def test_parts_are_powers_of_two_and_independent_of_the_row_count_within_a_class():
    for n, k in [(2560, 4096), (2560, 9728), (4096, 12288), (5120, 25600), (1024, 2048), (64, 512), (100, 256)]:
        few = {plan.rows_split(n, k, rows) for rows in (1, 8, 16)}
        many = {plan.rows_split(n, k, rows) for rows in (17, 33, 64)}
        assert len(few) == 1 and len(many) == 1  # one order of additions per class of row counts
        for parts, col_tiles in few | many:
            assert parts & (parts - 1) == 0 and col_tiles in (1, 2)


def test_a_projection_whose_consumer_adds_partial_sums_is_cut_over_k():
    """q/k/v in front of the decode attention that prepares its own operands: up to 16 rows two
    or four parts of 64 columns where that keeps the workgroups within the compute units (4B,
    8B: two; 32B: none); from 17 to 64 rows the split of a residual product (4B and 8B: four
    parts of 128 columns; 32B: two); a matrix that is not cut goes as `plan_projection` says."""
    for name, few, many in (("4b", (2, 1), (4, 2)), ("8b", (2, 1), (4, 2)), ("32b", None, (2, 2)),
                            ("1.7b", (4, 1), (4, 1))):
        hidden, q, kv, _ = SIZES[name]
        n = q + 2 * kv
        for rows in (1, 8, 16):
            c = plan.plan_summed_later(rows, n, hidden)
            if few is None:
                assert c == plan.plan_projection(rows, n, hidden)
            else:
                assert (c.kernel, c.parts, c.col_tiles) == ("rows", *few), (name, rows, c)
        for rows in (17, 40, 64):
            c = plan.plan_summed_later(rows, n, hidden)
            assert (c.kernel, c.parts, c.col_tiles) == ("rows", *many), (name, rows, c)
    # a head is never cut (nothing behind it adds), nor is a matrix with too little K per part
    for rows in (8, 40):
        assert plan.plan_summed_later(rows, VOCAB, 2560) == plan.plan_projection(rows, VOCAB, 2560)
        assert plan.plan_summed_later(rows, 6144, 256).parts == 1


def test_from_65_to_128_rows_the_products_that_are_added_later_stay_with_the_rows_kernel():
    """Two halves of the rows, each to workgroups of its own, with the choices of 64 rows: out,
    down and the q/k/v whose partial sums the attention adds.  Gate/up, the head and a q/k/v
    that must come whole go to the library, as does everything beyond 128 rows."""
    for name in SIZES:
        hidden, q, kv, inter = SIZES[name]
        for rows in (65, 100, 128):
            for n, k in ((hidden, q), (hidden, inter)):
                assert plan.plan_residual(rows, n, k) == plan.plan_residual(64, n, k), (name, rows, n, k)
            assert plan.plan_summed_later(rows, q + 2 * kv, hidden) == plan.plan_summed_later(64, q + 2 * kv, hidden)
            assert plan.plan_projection(rows, q + 2 * kv, hidden).kernel == "library"
            assert plan.plan_projection(rows, VOCAB, hidden).kernel == "library"
            assert plan.plan_gated(rows, inter, hidden, hidden).kernel == "library"
    assert plan.SPLIT_ROWS == 128 and plan.STREAM_ROWS == 64


def test_decode_attention_cuts_the_keys_of_few_long_requests_over_workgroups():
    """`ops.decode_cuts` is a pure function of the shape: up to 512 keys one workgroup per
    (token, head), as up to 767; beyond, powers of two of cuts of at least 192 keys while the workgroups stay
    within the compute units; none once the workgroups fill them."""
    from pylon_amd.kernels import ops

    for tokens in (1, 2, 8, 16, 64):
        for bound in (1, 64, 511, 512, 767):
            assert ops.decode_cuts(tokens, 8, bound, 256) == 1
    assert [ops.decode_cuts(1, 8, b, 256) for b in (768, 1024, 2048, 4096, 8192, 32768, 262144)] == [4, 4, 8, 16, 32, 32, 32]
    assert [ops.decode_cuts(8, 8, b, 256) for b in (1024, 2048, 4096, 262144)] == [4, 4, 4, 4]
    assert [ops.decode_cuts(16, 8, b, 256) for b in (1024, 8192)] == [2, 2]
    assert ops.decode_cuts(17, 8, 8192, 256) == 1 and ops.decode_cuts(64, 8, 8192, 256) == 1
    assert ops.decode_cuts(8, 8, None, 256) == 1
    for tokens in (1, 3, 5, 8, 13, 40):
        for heads in (1, 2, 8):
            for bound in (900, 5000, 70000):
                for units in (64, 256, 304):
                    cuts = ops.decode_cuts(tokens, heads, bound, units)
                    assert cuts & (cuts - 1) == 0 and 1 <= cuts <= 64
                    assert cuts == 1 or (tokens * heads * cuts <= units and cuts * 192 <= bound)
