"""Every route of the library under `pytest -m gpu`: the tests that exercise what a layer leaves unwritten until
first read (pending row resets, implicit appended columns, columns gathered from the weights, pending range
sums, zeros around generator windows) run again under each of the switches that select another route -- NaNs
in whatever is left unwritten, each "write at once" mode, the layer-by-layer path for small networks,
convolutions without row masks or windows, the full dense contraction.  The default route is what the other
test modules run; here the same test bodies are called with a switch set on the shared context."""
import pytest

from tests import test_gpu_mixed_sequences as seqs
from tests import test_gpu_parity as parity
from tests import test_gpu_small_chain as chain

pytestmark = pytest.mark.gpu

VARIANTS = {
    "poison_pending": ("poison_pending",),
    "eager_rows": ("eager_rows",),
    "eager_tail": ("eager_tail",),
    "eager_rows_and_tail": ("eager_rows", "eager_tail"),
    "eager_cols": ("eager_cols",),
    "everything_written_at_once": ("eager_rows", "eager_tail", "eager_cols"),
    "no_small_chain": ("no_small_chain",),
    "no_conv_mask": ("no_conv_mask",),
    "no_conv_boxes": ("no_conv_boxes",),
    "poison_without_conv_boxes": ("poison_pending", "no_conv_boxes"),
    "dense_affine": ("dense_affine",),
    "no_row_deltas": ("no_row_deltas",),
    "no_sum_shortcuts": ("no_sum_shortcuts",),
}


@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    nnv_amd.default_context()
    return nnv_amd


@pytest.fixture(scope="module")
def oracle():
    from oracle import nnv_oracle
    return nnv_oracle


@pytest.fixture(params=sorted(VARIANTS))
def route(request, nnv):
    """Sets the variant's switches on the shared context for one test and puts back what the environment says."""
    import os
    from nnv_amd._lib import SWITCH_ENV
    ctx = nnv.default_context()
    names = VARIANTS[request.param]
    for nm in names:
        ctx.set_switch(nm, True)
    try:
        yield request.param
    finally:
        for nm in names:
            ctx.set_switch(nm, os.environ.get(SWITCH_ENV[nm]) is not None)


@pytest.mark.parametrize("seed", [0, 3, 4, 7, 9])
def test_random_fc_sequences(route, nnv, oracle, seed):
    seqs.test_random_fc_sequences(nnv, oracle, seed)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_cnn_sequences(route, nnv, oracle, seed):
    seqs.test_random_cnn_sequences(nnv, oracle, seed)


@pytest.mark.parametrize("seed", [300, 305, 311, 317, 323])
def test_random_chains_of_convolutions(route, nnv, oracle, seed):
    seqs.test_random_chains_of_convolutions(nnv, oracle, seed)


@pytest.mark.parametrize("shapes,hidden", [(3, 300), (2, 1400)])
def test_arrays_of_boxes_that_share_their_half_widths(route, nnv, oracle, shapes, hidden):
    seqs.test_arrays_of_boxes_that_share_their_half_widths(nnv, oracle, shapes, hidden)


@pytest.mark.parametrize("spread,shapes", [(2e-3, 2), (2e-2, 3)])
def test_neighbouring_boxes_share_the_product_over_their_common_rows(route, nnv, oracle, spread, shapes):
    seqs.test_neighbouring_boxes_share_the_product_over_their_common_rows(nnv, oracle, spread, shapes, None)


@pytest.mark.parametrize("count,half_width", [(1, 3.0), (5, 0.3)])
def test_a_relu_on_top_of_a_relu_lists_its_rows_anew(route, nnv, oracle, count, half_width):
    seqs.test_a_relu_on_top_of_a_relu_lists_its_rows_anew(nnv, oracle, count, half_width)


def test_a_hint_about_the_next_fc_layer_changes_no_bit(route, nnv, oracle):
    seqs.test_a_hint_about_the_next_fc_layer_changes_no_bit(nnv, oracle, 64)


@pytest.mark.parametrize("then", ["relu", "batchnorm"])
def test_matrices_a_layer_leaves_unwritten_read_the_same_later(route, nnv, oracle, then):
    seqs.test_matrices_a_layer_leaves_unwritten_read_the_same_later(nnv, oracle, then)


@pytest.mark.parametrize("count", [1, 40])
def test_relu_steps_that_append_their_predicate_bounds_in_place(route, nnv, oracle, count):
    seqs.test_relu_steps_that_append_their_predicate_bounds_in_place(nnv, oracle, count)


def test_one_wide_set_through_the_tile_kernel(route, nnv, oracle):
    seqs.test_one_wide_set_through_the_tile_kernel(nnv, oracle, "relax-star-area")


@pytest.mark.parametrize("count", [1, 3])
def test_columns_left_unwritten_are_written_on_any_first_read(route, nnv, oracle, count):
    parity.test_columns_left_unwritten_are_written_on_any_first_read(nnv, oracle, count)


def test_relu_output_consumers_that_need_every_column(route, nnv, oracle):
    parity.test_relu_output_consumers_that_need_every_column(nnv, oracle)


def test_relu_output_whose_row_reset_is_still_pending(route, nnv, oracle):
    parity.test_relu_output_whose_row_reset_is_still_pending(nnv, oracle, 700, 300)


def test_fc_after_a_relu_that_kept_no_row(route, nnv, oracle):
    parity.test_fc_after_a_relu_that_kept_no_row(nnv, oracle)


def test_conv_reads_through_a_pending_row_reset(route, nnv, oracle):
    parity.test_conv_reads_through_a_pending_row_reset(nnv, oracle, 12, 12, 3, 8, 3, 3, 1, 1, 1, 30, 2)


def test_config1(route, nnv):
    parity.test_config1_full(nnv, "relax-star-area")


def test_config2(route, nnv, oracle):
    parity.test_config2_full(nnv, oracle, None)


def test_config3(route, nnv, oracle):
    parity.test_config3_full(nnv, oracle, None)


def test_config4_shrunk(route, nnv):
    parity.test_config4_shrunk(nnv)


def test_config5_shrunk_batched(route, nnv, oracle):
    parity.test_config5_shrunk_batched(nnv, oracle)


def test_small_network(route, nnv, oracle):
    chain.test_single_set(nnv, oracle, "relax-star-area", (8, 130, 70, 6), 0.02)
    chain.test_sets_of_a_chain_reach_feed_the_layer_kernels(nnv, oracle)
    chain.test_odd_sequences(nnv, oracle)
