"""The tiled product's choice of block shape and split, asked of the library without running a kernel (no GPU):
invariants over a sweep of sizes, and the decisions that measurements on the GPU settled."""
import itertools

import pytest

from sprout_lm_amd import ops



@pytest.fixture(autouse=True, scope="module")
def built_library():
    """The plan is asked of the compiled library, which needs hipcc where it is not built yet, but no GPU."""
    try:
        ops.library()
    except Exception as e:      # no compiler here: nothing to ask
        pytest.skip(f"the kernel library cannot be built or loaded here: {e}")


SHAPES = {(256, 256), (256, 128), (128, 128), (64, 64), (64, 256), (64, 128), (384, 256), (256, 160)}
PAIRED = {(256, 256), (256, 128), (128, 128), (64, 256), (64, 128), (384, 256)}    # an even number of tile columns a wave
ROTATING = {(256, 128), (128, 128), (64, 128)}


def sizes():
    tokens = [1, 5, 16, 17, 64, 65, 128, 200, 256, 264, 512, 777, 1024, 1100, 2048, 4096, 8192]
    rows = [64, 130, 896, 1152, 3584, 4608, 5120, 9728, 37888, 151936]
    depth = [64, 192, 896, 1088, 3584, 4864, 5120, 18944, 27648]
    return itertools.product(tokens, rows, depth)


@pytest.mark.parametrize("kind", [ops.PLAN_STORE, ops.PLAN_ACCUMULATE, ops.PLAN_GATED])
def test_plan_invariants(kind):
    for T, N, K in sizes():
        plan = ops.pipe_plan(kind, T, N, K)
        if N * K * 2 >= 1 << 32:      # a tile's offset into the weights has 32 bits: another kernel's product
            assert plan is None, (T, N, K)
            continue
        assert plan is not None, (T, N, K)          # K is a multiple of 64 everywhere here
        rows, cols, splits, waves = plan
        assert (rows, cols) in SHAPES and splits >= 1
        if kind == ops.PLAN_GATED:
            # gate and up rows alternate between a wave's tile columns (64 x 64 for up to 64 tokens is two waves with
            # two tile columns each; for more tokens it is four waves with one)
            assert (rows, cols) in PAIRED or T <= 64, (T, N, K, plan)
        if kind != ops.PLAN_ACCUMULATE:
            assert splits == 1, (T, N, K, plan)                  # only float atomics can join partial sums
        assert splits == 1 or K // 64 // splits >= 8, (T, N, K, plan)
        if T > 64:   # few tokens have shapes of their own
            assert (rows, cols) != (64, 256)


def test_products_the_kernel_does_not_take():
    assert ops.pipe_plan(ops.PLAN_STORE, 300, 100, 70) is None          # K is no multiple of 64
    assert ops.pipe_plan(ops.PLAN_STORE, 300, 100, 0) is None
    assert ops.pipe_plan(7, 300, 128, 128) is None
    assert ops.pipe_plan(ops.PLAN_ROTATING, 64, 1152, 896, 64) is None  # up to 64 tokens: the decode kernels rotate
    assert ops.pipe_plan(ops.PLAN_ROTATING, 300, 18 * 48, 896, 48) is None   # head sizes that are no multiple of 64


def test_rotating_epilogue_shapes():
    for T, (nq, nkv, hd, K) in itertools.product([65, 128, 256, 264, 512, 1024, 2048, 4096],
                                                  [(14, 2, 64, 896), (28, 4, 128, 3584), (40, 8, 128, 5120), (4, 4, 128, 256)]):
        plan = ops.pipe_plan(ops.PLAN_ROTATING, T, (nq + 2 * nkv) * hd, K, hd)
        assert plan is None or (plan[:2] in ROTATING and plan[2] == 1 and plan[3] in (4, 8)), (T, nq, nkv, hd, K, plan)


def test_decisions_that_measurements_settled():
    """(kind, T, N, K[, hd]) -> plan: each of these was timed against the other shapes with operands from memory."""
    settled = {
        (ops.PLAN_STORE, 2048, 37888, 3584): (256, 256, 1),       # fills the chip: the largest blocks
        (ops.PLAN_STORE, 2048, 4608, 3584): (256, 160, 1),        # 232 blocks where 256 x 256 make 144
        (ops.PLAN_ACCUMULATE, 2048, 5120, 27648): (256, 160, 1),  # 256 blocks where 256 x 256 make 160
        (ops.PLAN_ACCUMULATE, 2048, 3584, 3584): (256, 128, 1),
        (ops.PLAN_ACCUMULATE, 2048, 896, 4864): (128, 128, 2),
        (ops.PLAN_ACCUMULATE, 2048, 896, 896): (64, 64, 1),
        (ops.PLAN_GATED, 2048, 9728, 896): (384, 256, 1),
        (ops.PLAN_GATED, 256, 9728, 896): (128, 128, 1),
        (ops.PLAN_ROTATING, 2048, 1152, 896, 64): (128, 128, 1),
        (ops.PLAN_ROTATING, 1024, 1152, 896, 64): (64, 128, 1),
        (ops.PLAN_ROTATING, 512, 1152, 896, 64): None,            # 64 x 64 and a rotation kernel after it
        (ops.PLAN_ROTATING, 2048, 4608, 3584, 128): None,         # 256 x 160 and a rotation kernel after it
        (ops.PLAN_ROTATING, 1024, 4608, 3584, 128): (256, 128, 1),
        (ops.PLAN_ROTATING, 512, 4608, 3584, 128): (128, 128, 1),
        (ops.PLAN_ROTATING, 256, 4608, 3584, 128): (64, 128, 1),
    }
    for args, want in settled.items():
        got = ops.pipe_plan(*args)
        assert (got[:3] if got else None) == want, (args, got, want)


def test_kernel_tests_reach_every_block_shape():
    """The sizes that tests/test_gpu_kernels.py runs on the GPU, asked here for their plans: every block shape of the
    plain, the gated and the rotating product is reached by at least one of them."""
    import importlib
    kernels = importlib.import_module("tests.test_gpu_kernels")
    plain = {(rows, cols, waves, split) for rows, cols, waves, split in kernels.BLOCK_SHAPE_SIZES.values()}
    assert {(r, c) for r, c, _, _ in plain} == SHAPES - {(64, 256)} and {s for _, _, _, s in plain} == {False, True}
    for (accumulate, T, N, K), (rows, cols, waves, split) in kernels.BLOCK_SHAPE_SIZES.items():
        got = ops.pipe_plan(ops.PLAN_ACCUMULATE if accumulate else ops.PLAN_STORE, T, N, K)
        assert (got[0], got[1], got[3], got[2] > 1) == (rows, cols, waves, split), (T, N, K, got)
    rotating = set()
    for (T, nq, nkv, hd, K), shape in kernels.ROTATING_SHAPE_SIZES.items():
        got = ops.pipe_plan(ops.PLAN_ROTATING, T, (nq + 2 * nkv) * hd, K, hd)
        assert (got[0], got[1], got[3]) == shape, (T, nq, nkv, hd, K, got)
        rotating.add(shape[:2])
    assert rotating == ROTATING
    marks = [m for m in kernels.test_fused_gate_up_silu_and_normed_product.pytestmark
             if m.name == "parametrize" and m.args[0] == "T,I,K"]
    gated = {ops.pipe_plan(ops.PLAN_GATED, T, 2 * I, K)[:2] for T, I, K in marks[0].args[1] if T > 64 and K % 64 == 0}
    assert gated >= {(64, 128), (128, 128), (256, 128), (256, 256), (384, 256)}, gated


def test_blocks_are_numbered_so_that_every_tile_runs_once_and_the_xcds_share_them():
    """The tiled product's numbering of its blocks (block b runs on XCD b % 8): every (token tile, weight tile) is
    some block's, once; a weight tile of the whole eights lies on one XCD with all its token tiles (nobody else
    fetches it); and no XCD holds more blocks than its even share of the left-over tiles, rounded up."""
    for tiles_t in list(range(1, 20)) + [33, 64]:
        for tiles_n in list(range(1, 41)) + [148, 149, 593]:
            blocks = ops.pipe_tiles(tiles_t, tiles_n)
            assert len(blocks) % 8 == 0
            seen, per_xcd, home = {}, [0] * 8, {}
            for b, tile in enumerate(blocks):
                if tile is None:
                    continue
                t, n = tile
                assert 0 <= t < tiles_t and 0 <= n < tiles_n and tile not in seen, (tiles_t, tiles_n, b, tile)
                seen[tile] = b
                per_xcd[b % 8] += 1
                if n < tiles_n // 8 * 8:
                    assert home.setdefault(n, b % 8) == b % 8 == n % 8, (tiles_t, tiles_n, b, tile)
            assert len(seen) == tiles_t * tiles_n
            left = tiles_n % 8
            assert max(per_xcd) == tiles_n // 8 * tiles_t + -(-left * tiles_t // 8), (tiles_t, tiles_n, per_xcd)
    with pytest.raises(ops.KernelError):
        ops.pipe_tiles(0, 5)

