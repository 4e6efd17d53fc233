"""Which kernel a projection goes to is decided on the host from its sizes alone; the
decisions are checked here without a GPU."""

import pytest

from zig_ai_amd.kernels import ops


@pytest.mark.parametrize("M,N,K,plan", [
    (8, 2048, 2048, 4),          # few outputs: K in ranges until some 512 workgroups run
    (8, 2048, 8192, 4),
    (1, 64, 4096, 8),
    (8, 6144, 12288, 2),         # a wide model: outputs alone fill the chip, K is too long
    (3, 8192, 28672, 4),
    (16, 5136, 9216, 2),
    (2, 48, 8200, 0),            # no cut of 8200 is a multiple of 32: the product comes back
    (17, 2048, 2048, 0),         # more than a decode batch
    (8, 2048, 2052, 0),          # rows that do not start on 16-byte boundaries
])
def test_how_a_decode_product_reaches_the_stream(M, N, K, plan):
    assert ops.accumulate_plan(M, N, K, False) == plan


def test_every_plan_fits_the_kernel():
    """Whatever the sizes, a plan's ranges are what the decode kernel takes: no longer than a
    workgroup covers, and a multiple of 32 when K is cut."""
    for N in (16, 100, 2048, 5136, 6144, 8192, 65536, 200000):
        for K in range(8, 70000, 8):
            plan = ops.accumulate_plan(8, N, K, False)
            if plan == 0:
                continue
            assert (K + plan - 1) // plan <= ops.ROWS16_MAX_K_PER_WORKGROUP, (N, K, plan)
            assert plan == 1 or K % (plan * 32) == 0, (N, K, plan)


def test_the_kernel_that_runs_the_norm_covers_k_alone():
    assert ops.accumulate_plan(8, 2048, 2048, True) == 1
    assert ops.normed_rows_pay(8, 2048, 2048) and not ops.normed_rows_pay(8, 2048, 4608)
    assert ops.normed_rows_pay(16, 2048, 2048) and not ops.normed_rows_pay(17, 16384, 2048)


def test_when_the_output_projection_merges_the_context_ranges():
    """Few rows in few ranges: every workgroup of the projection merges its slice of every
    row, which pays while rows x ranges stays small."""
    from zig_ai_amd.kernels import ops
    assert ops.merged_rows_pay(1, 8) and ops.merged_rows_pay(3, 8) and ops.merged_rows_pay(8, 2)
    assert ops.merged_rows_pay(2, 2) and ops.merged_rows_pay(4, 4) and ops.merged_rows_pay(8, 3)
    assert not ops.merged_rows_pay(8, 4) and not ops.merged_rows_pay(5, 8) and not ops.merged_rows_pay(4, 8)
    assert ops.merged_rows_pay(1, 12) and ops.merged_rows_pay(2, 12) and not ops.merged_rows_pay(2, 16)
    assert not ops.merged_rows_pay(3, 12)
    assert not ops.merged_rows_pay(1, 1) and not ops.merged_rows_pay(1, 17) and not ops.merged_rows_pay(9, 2)



def test_where_the_kernel_for_17_to_64_rows_is_taken():
    """The feed-forward's fused first product up to 48 rows, up to 64 on a stream no wider
    than 1,024, for widths whose K is spans of 512 (at least two) up to 4096; the mixer's
    closing product of such a step adds itself to the stream (through the library, see the
    next test; this package's kernel, where the library has nothing, when K is short and
    enough workgroups come of it)."""
    assert ops.rows64_swiglu_fusable(17, 2048) and ops.rows64_swiglu_fusable(32, 1024)
    assert ops.rows64_swiglu_fusable(33, 1024) and ops.rows64_swiglu_fusable(64, 1024)
    assert not ops.rows64_swiglu_fusable(65, 1024) and not ops.rows64_swiglu_fusable(49, 1536)
    assert ops.rows64_swiglu_fusable(20, 1536) and ops.rows64_swiglu_fusable(24, 4096)
    assert not ops.rows64_swiglu_fusable(16, 2048)      # the decode kernel's
    assert ops.rows64_swiglu_fusable(48, 2048)
    assert not ops.rows64_swiglu_fusable(49, 2048)      # measured no faster than the library's path
    assert not ops.rows64_swiglu_fusable(20, 512) and not ops.rows64_swiglu_fusable(20, 1280)
    assert not ops.rows64_swiglu_fusable(20, 4608)
    assert ops.rows64_add_splits(2048, 2048) == 2       # 32 tiles x 2 ranges of 1,024
    assert ops.rows64_add_splits(2048, 4096) == 4
    assert ops.rows64_add_splits(2048, 8192) == 0       # the library's ranges of K are faster
    assert ops.rows64_add_splits(1024, 1024) == 0       # 16 workgroups: too few
    assert ops.rows64_add_splits(4096, 1024) == 1
    assert ops.rows64_add_splits(2048, 1280) == 0       # no cut into spans of 512
    for K in range(512, 9000, 256):
        for N in (1024, 2048, 4096):
            ks = ops.rows64_add_splits(N, K)
            assert ks == 0 or ops.rows64_takes(32, K, ks)


def test_where_the_library_adds_a_product_to_the_stream_itself():
    """Many rows (beyond those whose K the library gets in ranges): only with a long K, the
    feed-forward's closing product.  Few rows (17 to 64): only with a short K, a mixer's
    closing product, and only where a feed-forward that runs its norm itself can follow on a
    stream of that width.  Elsewhere the product comes back and the next norm adds it."""
    assert ops.library_adds(2048, 2048, 8192) and ops.library_adds(1025, 1024, 4608)
    assert ops.library_adds(4096, 2560, 10752)
    assert not ops.library_adds(2048, 2048, 2048)          # the mixers' closing products
    assert not ops.library_adds(1024, 2048, 8192)          # K in ranges instead
    assert not ops.library_adds(2048, 2048, 4100)          # rows that do not start on 16 bytes
    for M in (17, 64, 512, 1024):
        assert not ops.library_adds(M, 2048, 8192)
    # few rows
    for M in (17, 24, 32):
        assert ops.library_adds(M, 2048, 2048) and ops.library_adds(M, 1024, 1024)
        assert ops.library_adds(M, 2048, 1024)
    for M in (33, 48, 64):
        assert ops.library_adds(M, 1024, 1024) and ops.library_adds(M, 2048, 2048) == (M <= 48)
    for M in (16, 65, 128, 512):
        assert not ops.library_adds(M, 1024, 1024)
    assert not ops.library_adds(24, 1280, 1024)            # no fused feed-forward at that width
    assert not ops.library_adds(24, 2048, 4096)            # a long K stays in ranges


def test_the_batch_sizes_that_recordings_are_kept_for():
    """A decode batch without a recording of its own is filled up to 1, 2, 4, 8, 16 requests
    or, beyond, to a multiple of 8: never by more than 7 rows."""
    from zig_ai_amd.engine.runner import ModelRunner
    sizes = [ModelRunner.padded_size(n) for n in range(1, 70)]
    assert sizes[:17] == [1, 2, 4, 4, 8, 8, 8, 8, 16, 16, 16, 16, 16, 16, 16, 16, 24]
    assert all(0 <= s - n <= 7 for n, s in zip(range(1, 70), sizes))
    assert all(s % 8 == 0 for s in sizes[16:]) and sizes[63] == 64 and sizes[64] == 72
