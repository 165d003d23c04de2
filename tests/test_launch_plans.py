"""Launch plans without a GPU: lutgemm_describe_plan is pure host arithmetic, so the
planner's invariants are checked here over the benchmark shapes and a few thousand
random ones.  What a kernel relies on (and cannot check itself):
  look-up kernel   the ranges cover every (tile, set) item exactly once, none is empty,
                   and no output tile receives more than 40 contributions (the count field
                   of an accumulator word, lutgemm_common.h);
  matrix cores     the K-slices cover every step, none is empty, each is a whole number of
                   eight-step rounds, and there are at most 32 of them per tile."""
import ctypes
import os
import random

import pytest

LOOKUP, MATRIX_CORE = 0, 1
ROWWISE, BLOCK_F16, BLOCK_U16, BLOCK_I8, UNIFORM = range(5)
MAX_CONTRIB = 40
MAX_SLICES = 32


@pytest.fixture(scope="module")
def lib():
    from shiftaddllm_amd import native
    if not os.path.exists(native.KERNEL_LIB):
        from shiftaddllm_amd import build
        build.build_kernel_library()
    return native.cabi()


def describe(lib, fmt, N, K, nb, groups, M):
    from shiftaddllm_amd import native
    plan = native.Plan()
    rc = lib.lutgemm_describe_plan(fmt, N, K, nb, groups, M, ctypes.byref(plan))
    return rc, plan


def check_plan(p, N, K, M):
    assert p.workgroups >= 1 and p.row_chunks == -(-M // p.rows_per_pass)
    if p.kernel == LOOKUP:
        assert p.tile_columns in (256, 512) and p.tiles == -(-N // p.tile_columns) and p.k_units == -(-K // 256)
        if p.tile_columns == 512:      # twin items: one row, every range of at least two of them unless there is only one
            assert p.rows_per_pass == 1 and M == 1
        total = p.tiles * p.k_units
        a, b, n_long, n = p.items_per_long_range, p.items_per_short_range, p.long_ranges, p.ranges
        assert a >= b >= 1 and 1 <= n_long <= n and p.workgroups == n * p.row_chunks
        starts = [min(r, n_long) * a + max(r - n_long, 0) * b for r in range(n + 1)]
        assert starts[n] >= total, "ranges must cover every item"
        assert starts[n - 1] < total, "no range may be empty"
        # contributions per tile = ranges overlapping its k_units items
        bounds = starts[:n] + [total]
        worst, split = 0, False
        r = 0
        for t in range(p.tiles):
            lo, hi = t * p.k_units, (t + 1) * p.k_units
            while bounds[r + 1] <= lo:
                r += 1
            c, rr = 1, r
            while bounds[rr + 1] < hi:
                rr += 1
                c += 1
            worst = max(worst, c)
            split = split or c > 1
        assert worst <= MAX_CONTRIB, worst
        assert bool(p.needs_workspace) >= split, "a tile shared between ranges needs accumulator words"
    else:
        assert p.tiles == -(-N // 64) and p.k_units == K // 128
        assert p.rows_per_pass in (16, 32)
        assert 1 <= p.k_slices <= MAX_SLICES and p.units_per_slice % 8 == 0
        assert p.k_slices * p.units_per_slice >= p.k_units, "slices must cover every K-step"
        assert (p.k_slices - 1) * p.units_per_slice < p.k_units, "no slice may be empty"
        assert p.workgroups == p.tiles * p.k_slices * p.row_chunks
        assert bool(p.needs_workspace) == (p.k_slices > 1)


BENCH_SHAPES = [(3072, 768), (4096, 4096), (11008, 4096), (4096, 11008), (5120, 5120), (13824, 5120), (5120, 13824),
                (8192, 8192), (28672, 8192), (8192, 28672), (1024, 8192), (22016, 4096), (32000, 4096)]


@pytest.mark.parametrize("N,K", BENCH_SHAPES)
def test_benchmark_shapes_every_bit_width_and_batch(lib, N, K):
    for nb in (1, 2, 3, 4):
        for M in (1, 2, 3, 4, 8, 16, 17, 32, 33, 64):
            rc, p = describe(lib, ROWWISE, N, K, nb, K // 128, M)
            assert rc == 0, (N, K, nb, M, rc)
            check_plan(p, N, K, M)
        for fmt in (BLOCK_F16, BLOCK_U16, BLOCK_I8):
            for M in (1, 2, 5):
                rc, p = describe(lib, fmt, N, K, nb, 8, M)
                assert rc == 0 and p.kernel == LOOKUP
                check_plan(p, N, K, M)


def test_which_kernel_takes_what(lib):
    # one row: always the look-up kernel; three rows and more of an eligible problem: matrix cores
    assert describe(lib, ROWWISE, 4096, 4096, 3, 32, 1)[1].kernel == LOOKUP
    assert describe(lib, ROWWISE, 4096, 4096, 3, 32, 3)[1].kernel == MATRIX_CORE
    assert describe(lib, ROWWISE, 4096, 4096, 3, 32, 32)[1].rows_per_pass == 32
    # two rows: matrix cores on short sign streams, the look-up kernel (both rows per pass) on long ones
    assert describe(lib, ROWWISE, 4096, 4096, 3, 32, 2)[1].kernel == MATRIX_CORE
    big = describe(lib, ROWWISE, 28672, 8192, 4, 64, 2)[1]
    assert big.kernel == LOOKUP and big.rows_per_pass == 2 and big.row_chunks == 1
    # not eligible for the matrix cores: K not a multiple of 128, groups of 32 inputs, other formats
    assert describe(lib, ROWWISE, 1024, 288, 3, 9, 8)[1].kernel == LOOKUP
    assert describe(lib, ROWWISE, 1024, 1024, 3, 32, 8)[1].kernel == LOOKUP
    assert describe(lib, UNIFORM, 1024, 1024, 3, 8, 8)[1].kernel == LOOKUP
    # the 70B shapes at one row run two workgroups per CU with unequal ranges
    p = describe(lib, ROWWISE, 28672, 8192, 4, 64, 1)[1]
    assert p.ranges == 512 and p.long_ranges == 256 and p.items_per_long_range > p.items_per_short_range
    # the 7B gate|up pair as one problem at eight rows: two K-slices per tile (more workgroups than are resident)
    assert describe(lib, ROWWISE, 22016, 4096, 3, 32, 8)[1].k_slices == 2


def test_random_shapes(lib):
    rng = random.Random(1234)
    seen = {LOOKUP: 0, MATRIX_CORE: 0}
    for i in range(4000):
        if i % 2:                                    # shapes the matrix-core kernel takes at three rows and more
            K = 128 * rng.randint(1, 300)
            N = 16 * rng.randint(1, 2250)
        else:
            K = 32 * rng.randint(1, 1200)
            N = 4 * rng.randint(1, 9000)
        nb = rng.randint(1, 4)
        M = rng.choice((1, 1, 1, 2, 3, 4, 7, 16, 17, 40, 100))
        divisors = [g for g in ((128, 256, 512, K) if i % 2 else (32, 64, 96, 128, 256, 512, K)) if K % g == 0]
        gs = rng.choice(divisors)
        rc, p = describe(lib, ROWWISE, N, K, nb, K // gs, M)
        if rc != 0:
            assert rc == -3, (N, K, nb, gs, M, rc)      # LUTGEMM_EUNSUP: beyond the exact-division bounds
            continue
        check_plan(p, N, K, M)
        seen[p.kernel] += 1
    assert seen[LOOKUP] > 500 and seen[MATRIX_CORE] > 100


def test_bad_arguments(lib):
    from shiftaddllm_amd import native
    plan = native.Plan()
    assert lib.lutgemm_describe_plan(ROWWISE, 4096, 4096, 3, 32, 1, None) == -1
    assert lib.lutgemm_describe_plan(9, 4096, 4096, 3, 32, 1, ctypes.byref(plan)) == -1
    assert lib.lutgemm_describe_plan(ROWWISE, 4096, 4100, 3, 32, 1, ctypes.byref(plan)) == -1   # K % 32
    assert lib.lutgemm_describe_plan(ROWWISE, 4096, 4096, 5, 32, 1, ctypes.byref(plan)) == -1   # bit planes
    assert lib.lutgemm_describe_plan(ROWWISE, 4096, 4096, 3, 32, 0, ctypes.byref(plan)) == -1   # rows


def test_tuning_options_change_plans_and_keep_their_invariants(lib):
    """lutgemm_set_option: every option changes the plan it is documented to change, the plans stay
    legal, and a negative value restores the start value."""
    from shiftaddllm_amd import native
    opt = native.OPTIONS
    start = {k: lib.lutgemm_get_option(v) for k, v in opt.items()}
    try:
        # workgroups a look-up launch aims for
        _, base = describe(lib, ROWWISE, 11008, 4096, 3, 32, 1)
        assert base.workgroups <= 256
        assert lib.lutgemm_set_option(opt["TARGET_BLOCKS"], 512) == 0
        _, p = describe(lib, ROWWISE, 11008, 4096, 3, 32, 1)
        assert 256 < p.workgroups <= 512
        check_plan(p, 11008, 4096, 1)
        lib.lutgemm_set_option(opt["TARGET_BLOCKS"], -1)
        # share of the first-dispatched workgroup: 50 = equal ranges
        _, base = describe(lib, ROWWISE, 28672, 8192, 4, 64, 1)
        assert base.items_per_long_range > base.items_per_short_range
        lib.lutgemm_set_option(opt["FIRST_SHARE"], 50)
        _, p = describe(lib, ROWWISE, 28672, 8192, 4, 64, 1)
        assert p.items_per_long_range == p.items_per_short_range
        check_plan(p, 28672, 8192, 1)
        lib.lutgemm_set_option(opt["FIRST_SHARE"], -1)
        # rows from which the matrix-core kernel takes over
        lib.lutgemm_set_option(opt["MFMA_MIN_M"], 2)
        _, p = describe(lib, ROWWISE, 8192, 8192, 4, 64, 2)
        assert p.kernel == MATRIX_CORE
        lib.lutgemm_set_option(opt["MFMA_MIN_M"], 1000)
        _, p = describe(lib, ROWWISE, 8192, 8192, 4, 64, 16)
        assert p.kernel == LOOKUP and p.rows_per_pass == 4
        check_plan(p, 8192, 8192, 16)
        lib.lutgemm_set_option(opt["MFMA_MIN_M"], -1)
        # workgroups aimed at per matrix-core launch
        lib.lutgemm_set_option(opt["MFMA_BLOCKS"], 1024)
        _, p = describe(lib, ROWWISE, 8192, 8192, 4, 64, 16)
        assert p.kernel == MATRIX_CORE and p.k_slices == 8
        check_plan(p, 8192, 8192, 16)
        lib.lutgemm_set_option(opt["MFMA_BLOCKS"], -1)
        assert lib.lutgemm_set_option(99, 1) == -1 and lib.lutgemm_get_option(-2) == -1
    finally:
        for k, v in opt.items():
            lib.lutgemm_set_option(v, -1)
    assert {k: lib.lutgemm_get_option(v) for k, v in opt.items()} == start


# ---- chained launches: the forward-progress argument as host arithmetic ---------------------------

def _chain_problem(base, N, K, nb, x, out, M=1, x_tag=0, gate_tag=0, out_tag=0, gate=None, norm=None, overwrite=0):
    from shiftaddllm_amd import native
    f = native.FusedProblem(base, base + 0x100000, x, out, N, K, nb, K // 128, M, overwrite, norm, gate, 1e-5)
    return native.ChainProblem(f, x_tag, gate_tag, out_tag)


def _decoder_block_chain(hidden, inter, nbs, M=1):
    """o_proj -> gate, up -> down_proj -> q, k, v of the next block (dummy, never dereferenced addresses)."""
    A = 0x10000000
    att, xt, gt, ut, q, k, v, w = (A + i * 0x1000000 for i in range(1, 9))
    return [_chain_problem(A, hidden, hidden, nbs[0], att, xt, M, out_tag=1),
            _chain_problem(A, inter, hidden, nbs[1], xt, gt, M, x_tag=1, out_tag=2, norm=w, overwrite=1),
            _chain_problem(A, inter, hidden, nbs[2], xt, ut, M, x_tag=1, out_tag=3, norm=w, overwrite=1),
            _chain_problem(A, hidden, inter, nbs[3], ut, xt, M, x_tag=3, gate_tag=2, out_tag=4, gate=gt),
            _chain_problem(A, hidden, hidden, nbs[4], xt, q, M, x_tag=4, norm=w, overwrite=1),
            _chain_problem(A, hidden // 4, hidden, nbs[5], xt, k, M, x_tag=4, norm=w, overwrite=1),
            _chain_problem(A, hidden // 4, hidden, nbs[6], xt, v, M, x_tag=4, norm=w, overwrite=1)]


def _describe_chain(lib, problems, workgroups):
    from shiftaddllm_amd import native
    arr = (native.ChainProblem * len(problems))(*problems)
    plan = native.ChainPlan()
    rc = lib.lutgemm_describe_chain_plan(len(problems), arr, workgroups, ctypes.byref(plan))
    return rc, plan


@pytest.mark.parametrize("workgroups", [64, 256, 512])
@pytest.mark.parametrize("hidden,inter,nbs,M", [(4096, 11008, (3,) * 7, 1), (4096, 11008, (2, 4, 3, 3, 4, 2, 3), 2),
                                                (1024, 2688, (3, 2, 4, 3, 2, 3, 4), 1), (8192, 28672, (4,) * 7, 1)])
def test_chain_plans_cannot_starve_a_producer(lib, workgroups, hidden, inter, nbs, M):
    """Workgroup w of a chained launch takes units w, w + G, w + 2G, ... in that order, and a unit waits
    only for units of problems that come earlier in the call.  Checked on the plans: units are numbered
    problem by problem without gaps, every problem a unit waits for has all its units below the
    waiter's first unit, stages never decrease, and a unit's items fit one activation window.  Then the
    schedule is simulated: at every moment the unfinished unit with the smallest number is at the
    head of its workgroup's queue and everything it waits for has finished."""
    problems = _decoder_block_chain(hidden, inter, nbs, M)
    rc, plan = _describe_chain(lib, problems, workgroups)
    assert rc == 0
    n = len(problems)
    G = plan.workgroups
    assert 1 <= G <= workgroups
    first = [plan.first_unit[i] for i in range(n)]
    count = [plan.unit_count[i] for i in range(n)]
    stage = [plan.stage[i] for i in range(n)]
    assert first[0] == 0 and all(first[i + 1] == first[i] + count[i] for i in range(n - 1))
    assert plan.units == first[-1] + count[-1] and all(c >= 1 for c in count)
    assert stage == sorted(stage) and stage == [0, 1, 1, 2, 3, 3, 3]
    assert all(1 <= plan.items_per_unit[i] <= 16 for i in range(n))
    waits_for = {1: [0], 2: [0], 3: [1, 2], 4: [3], 5: [3], 6: [3]}          # by construction of the block
    for i, ps in waits_for.items():
        for p in ps:
            assert first[p] + count[p] <= first[i], "a producer's units all come before its consumers'"
    # simulate: units finish in some order compatible with "a unit runs when it is at the head of its
    # workgroup's queue and its producers are done"; the smallest unfinished unit must always be runnable
    owner_of = lambda u: u % G
    problem_of = lambda u: max(i for i in range(n) if first[i] <= u)
    done = [False] * plan.units
    head = list(range(min(G, plan.units)))                                    # next unit of every workgroup
    for step in range(plan.units):
        u = step                                                               # the smallest unfinished unit
        assert head[owner_of(u)] == u, "its workgroup has finished everything before it"
        for p in waits_for.get(problem_of(u), []):
            assert all(done[first[p]:first[p] + count[p]])
        done[u] = True
        head[owner_of(u)] = u + G


def test_chain_plan_validation_on_the_host(lib):
    A = 0x10000000
    x, t1, t2, o = A + 0x1000000, A + 0x2000000, A + 0x3000000, A + 0x4000000
    ok = [_chain_problem(A, 512, 512, 3, x, t1, out_tag=1, overwrite=1),
          _chain_problem(A, 512, 512, 3, t1, t2, x_tag=1, out_tag=2, overwrite=1)]
    rc, plan = _describe_chain(lib, ok, 512)
    assert rc == 0 and plan.stage[0] == 0 and plan.stage[1] == 1 and plan.needs_workspace in (0, 1)
    # the consumer listed before its producer
    assert _describe_chain(lib, ok[::-1], 512)[0] == -1
    # two writers of one plain row; of one tagged row without an ordering wait
    assert _describe_chain(lib, [_chain_problem(A, 512, 512, 3, x, o), _chain_problem(A, 512, 512, 3, x, o)], 512)[0] == -1
    assert _describe_chain(lib, [_chain_problem(A, 512, 512, 3, x, t1, out_tag=1),
                                 _chain_problem(A, 512, 512, 3, x, t1, out_tag=2)], 512)[0] == -1
    # accumulating into a row right behind its writer
    assert _describe_chain(lib, [_chain_problem(A, 512, 512, 3, x, t1, out_tag=1),
                                 _chain_problem(A, 512, 512, 3, t1, t1, x_tag=1, out_tag=2)], 512)[0] == -1
    # tags out of range, rows beyond the limit, a tagged norm row wider than 8192
    assert _describe_chain(lib, [_chain_problem(A, 512, 512, 3, x, t1, out_tag=70000)], 512)[0] == -1
    assert _describe_chain(lib, [_chain_problem(A, 512, 512, 3, x, o, M=8)], 512)[0] == -3
    assert _describe_chain(lib, [_chain_problem(A, 512, 16384, 3, t1, o, x_tag=5, norm=x)], 512)[0] == -3
    # units of more than sixteen items would not fit one activation window: the stage takes more rounds
    rc, plan = _describe_chain(lib, [_chain_problem(A, 8192, 8192, 3, x, o)], 8)
    assert rc == 0 and plan.workgroups == 8 and plan.items_per_unit[0] <= 16 and plan.unit_count[0] >= 64


def test_pow2_plan_takes_the_block_scaled_kernel_for_few_rows_of_large_matrices():
    """lutgemm_describe_pow2_plan: up to 5 rows from 48 MB of sign words on and up to 8 rows from 96 MB
    on run block-scaled (kernel 2) in chunks of 5 or 8 rows; everything else is planned as
    lutgemm_gemv_rowwise_f16 plans it.  Option BLOCK_SCALED: 0 never, 2 wherever the kernel applies."""
    import ctypes
    from shiftaddllm_amd import native
    lib = native.cabi()
    which = native.OPTIONS["BLOCK_SCALED"]

    def plan(N, K, nb, M, group=128):
        p = native.Plan()
        assert lib.lutgemm_describe_pow2_plan(N, K, nb, K // group, M, ctypes.byref(p)) == 0
        return p

    def same_as_fp16(N, K, nb, M, group=128):
        a, b = plan(N, K, nb, M, group), native.Plan()
        assert lib.lutgemm_describe_plan(0, N, K, nb, K // group, M, ctypes.byref(b)) == 0
        return bytes(a) == bytes(b)

    try:
        lib.lutgemm_set_option(which, 1)
        p = plan(28672, 8192, 4, 4)
        assert (p.kernel, p.rows_per_pass, p.row_chunks, p.tile_columns, p.tiles) == (2, 5, 1, 64, 448)
        assert p.k_units == 64 and p.k_slices * p.units_per_slice >= 64 and p.workgroups == 448 * p.k_slices
        assert p.needs_workspace == (p.k_slices > 1)
        assert plan(28672, 8192, 2, 5).kernel == 2            # 56 MB
        p = plan(28672, 8192, 4, 8)                           # 112 MB
        assert (p.kernel, p.rows_per_pass) == (2, 8)
        assert same_as_fp16(28672, 8192, 2, 8)                # 8 rows want 96 MB
        assert same_as_fp16(28672, 8192, 4, 16)               # more than 8 rows: the fp16 kernel
        assert same_as_fp16(4096, 4096, 3, 4)                 # small matrix
        assert same_as_fp16(28672, 8192, 4, 1) and same_as_fp16(28672, 8192, 4, 2)   # look-up kernel
        assert same_as_fp16(28672, 8192, 4, 4, group=32)      # groups of 32: not a matrix-core shape
        lib.lutgemm_set_option(which, 2)
        p = plan(4096, 4096, 3, 33)
        assert (p.kernel, p.rows_per_pass, p.row_chunks) == (2, 16, 3)
        assert same_as_fp16(4096, 4096, 3, 2)
        lib.lutgemm_set_option(which, 0)
        assert same_as_fp16(28672, 8192, 4, 4)
    finally:
        lib.lutgemm_set_option(which, -1)
