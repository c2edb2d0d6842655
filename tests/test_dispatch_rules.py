"""The rules that choose a kernel's shape from the sizes: pure functions, tested without a GPU."""
from torchless_rs_amd.kernels import ops


def test_mid_splits_fit():
    for M in (17, 64, 128):
        for N in (72, 4096, 6144, 28672, 32000):
            for K in (48, 256, 1000, 4096, 14336):
                S = ops.mid_splits(M, N, K, 256)
                if K % ops.RING_K == 0:                  # the ring kernel: every slice has a stage of 128 k at least
                    assert 1 <= S <= max(1, K // 128) and S <= 16, (M, N, K, S)
                    assert -(-N // 128) * S <= 256 or S == 1, (M, N, K, S)      # one round of workgroups
                else:                                    # gemm_mid: powers of two, a step of 256 k at least each
                    steps = -(-K // 256)
                    assert S >= 1 and S & (S - 1) == 0, (M, N, K, S)
                    assert S <= max(1, steps) and S <= 16, (M, N, K, S)
    # the 7B sizes: narrow outputs are cut to one round of workgroups on 256 compute units, the wide one is not cut
    assert ops.mid_splits(64, 4096, 4096, 256) == 8 and ops.mid_splits(64, 6144, 4096, 256) == 5
    assert ops.mid_splits(128, 4096, 14336, 256) == 8 and ops.mid_splits(64, 28672, 4096, 256) == 1
    assert ops.mid_splits(64, 5120, 14336, 256) == 6 and ops.mid_splits(64, 5120, 14336, units=320) == 8
    assert ops.mid_splits(64, 4096, 256, 256) == 1          # two stages: nothing to cut
    assert ops.mid_splits(20, 72, 48, 256) == 1             # (gemm_mid) one step of K: nothing to cut
    assert ops.mid_splits(64, 4096, 4104, 256) == 8         # (gemm_mid) K no multiple of 128: 64 x 8 workgroups
    assert ops.own_rows(4096) == ops.MID_ROWS and ops.own_rows(4104) == ops.LIBRARY_ROWS


def test_decode_splits_follow_batch_and_length():
    assert ops.decode_groups(8, 32, 8) == 64 and ops.decode_groups(1, 34, 2) == 4      # 17 heads a group: two tiles
    # heads of 128 (and 64): the kernel that stages pages in LDS, two workgroups a compute unit
    assert ops.decode_workgroups_per_unit(128) == 2 and ops.decode_workgroups_per_unit(64) == 2
    assert ops.decode_workgroups_per_unit(256) == 1 and ops.decode_workgroups_per_unit(96) == 1
    assert ops.decode_workgroups_per_unit(32) == 4 and ops.decode_workgroups_per_unit(48) == 2
    assert ops.decode_splits(64, 32, 8, 32, 256, 128) == 1            # enough workgroups without a cut
    assert ops.decode_splits(32, 32, 8, 65, 256, 128) == 2            # 256 groups: two parts are two workgroups a unit
    assert ops.decode_splits(8, 32, 8, 65, 256, 128) == 8             # 64 groups: eight parts fill the round of 512
    assert ops.decode_splits(16, 32, 8, 65, 256, 128) == 4
    assert ops.decode_splits(3, 32, 8, 65, 256, 128) == 17            # 24 groups: at least four pages a part
    assert ops.decode_splits(20, 32, 8, 65, 256, 128) == 3            # 160 groups: 480 workgroups in one round
    assert ops.decode_splits(1, 32, 8, 64, 256, 128) == 16            # at least four pages a part
    assert ops.decode_splits(1, 32, 8, 513, 256, 128) == 57           # a long context: one round of workgroups, 9 pages each
    assert ops.decode_splits(8, 32, 8, 65, 128, 128) == 4             # by the device's compute units
    assert ops.decode_splits(8, 32, 8, 65, 256, 96) == 4              # a head size of the kernel that reads into registers: one a unit
    assert ops.decode_splits(8, 32, 8, 65, 256, 64) == 8 and ops.decode_splits(32, 16, 4, 64, 256, 32) == 8   # small heads: more workgroups a unit
    assert ops.decode_splits(1, 32, 8, 1, 256, 128) == 1
    for B in (1, 3, 8, 64):
        for pages in (1, 4, 5, 64, 1100):
            S = ops.decode_splits(B, 32, 8, pages, 256, 128)
            assert 1 <= S <= max(1, -(-pages // ops.SPLIT_PAGES))


def test_rows_choose_the_kernel():
    """Which product runs follows from the number of rows alone: the fused kernels up to 16, the one
    that shares activations to MID_ROWS, cut into partial sums where few channels leave the chip idle."""
    import torch
    from torchless_rs_amd.parts.linear import Linear
    lin = Linear(torch.zeros(4096, 4096, dtype=torch.bfloat16))
    rows = lambda m: torch.zeros(m, 4096, dtype=torch.bfloat16)
    assert [lin.mid(rows(m)) for m in (1, 16, 17, ops.MID_ROWS, ops.MID_ROWS + 1)] == [False, False, True, True, False]
    assert not lin.mid(torch.zeros(32, 4096))                        # float32 rows: the plain kernel
    assert [lin.own_kernels(m) for m in (1, 64, 128, 129)] == [True, True, True, False]
    odd = Linear(torch.zeros(96, 4104, dtype=torch.bfloat16))        # K no multiple of 128: the library from 65 rows on
    assert [odd.mid(torch.zeros(m, 4104, dtype=torch.bfloat16)) for m in (17, 64, 65)] == [True, True, False]
    assert [odd.own_kernels(m) for m in (64, 65)] == [True, False]


def test_prefill_layout_cuts_long_blocks_of_small_launches_into_runs():
    """The host's layout for the multi-token attention of a step with fewer workgroups than compute
    units: every block's keys are covered once, by one entry or by consecutive runs, no run shorter
    than the rule says, no more runs than there are units for, the dearest entries last."""
    import itertools

    def check(n_new, before, window, nq, units):
        laid = ops.prefill_layout(n_new, before, window, nq, units)
        blocks = [(b, t) for b, n in enumerate(n_new) for t in range(-(-n // 128))]
        if laid is None:
            return None
        entries, cut, n_blocks = laid
        assert n_blocks == len(blocks) and len(blocks) * nq <= units
        run = ops.PREFILL_CUT_TILES * (1 if len(blocks) * nq * 2 <= units else 2)
        most = min(ops.PREFILL_MAX_WAYS, 2 * units // (len(blocks) * nq))
        ways_of = {(b, t): w for b, t, w in cut}
        assert ways_of and all(2 <= w <= most for w in ways_of.values())
        tiles_of = {}
        for bt in blocks:
            b, t = bt
            lo_pos = before[b] + 128 * t
            hi_pos = before[b] + min(128 * (t + 1), n_new[b]) - 1
            first = max(0, lo_pos - window + 1) // 64 if window else 0
            last = hi_pos // 64
            tiles_of[bt] = last - first + 1
            mine = sorted((lo, w & 0xffffff, (w >> 24) & 7, ((w >> 27) & 7) + 1 if w >> 30 else 0)
                          for eb, et, lo, w in entries if (eb, et) == bt)
            if bt not in ways_of:
                assert mine == [(0, 0, 0, 0)] and (last - first + 1) // run < 2
                continue
            assert [m[2] for m in mine] == list(range(ways_of[bt])) and {m[3] for m in mine} == {ways_of[bt]}
            assert mine[0][0] == first and mine[-1][1] == last + 1
            assert all(x[1] == y[0] for x, y in zip(mine, mine[1:])) and all(m[1] - m[0] >= run for m in mine)
            assert ways_of[bt] == min(most, (last - first + 1) // run)
        cost = [(w & 0xffffff) - lo if w >> 30 else tiles_of[(eb, et)] for eb, et, lo, w in entries]
        assert cost == sorted(cost)                  # workgroups start from the end of the table: the dearest first
        assert len(entries) == len(blocks) + sum(w - 1 for w in ways_of.values())
        return laid

    # the cases of the design notes: few rows over a long context are cut, a launch that fills the device is not
    assert check([200], [8192], None, 32, 256) is not None
    assert check([256], [32768], None, 32, 256)[1] == [(0, 0, 8), (0, 1, 8)]
    assert check([512], [4096], None, 32, 256)[1] == [(0, t, 4) for t in range(4)]
    assert check([600], [35000], None, 32, 256)[1] == [(0, t, 3) for t in range(5)]      # 160 workgroups: three runs each
    assert check([100], [32768], None, 32, 256) is not None
    assert ops.prefill_layout([2048], [0], None, 32, 256) is None and ops.prefill_layout([1024], [0], None, 32, 256) is None
    assert ops.prefill_layout([100], [100], None, 4, 256) is None                           # nothing long
    assert ops.prefill_layout([128] * 9, [50000] * 9, None, 32, 256) is None                # 288 workgroups
    assert check([128] * 8, [50000] * 8, None, 32, 256)[1] == [(b, 0, 2) for b in range(8)]
    # a window bounds the tiles of a block: 4,096 positions are 64 tiles and the block's own two
    assert check([128], [100000], 4096, 32, 256)[1] == [(0, 0, 8)]
    assert ops.prefill_layout([128], [100000], 512, 32, 256) is None                        # ten tiles
    for n_new, before, window, nq, units in itertools.product(
            ([1], [129], [300, 5], [128, 128, 700], [1500]), ([0], [63], [5000], [70000]), (None, 70, 4096),
            (1, 4, 32), (8, 256, 1024)):
        before = (before * len(n_new))[:len(n_new)]
        check(n_new, before, window, nq, units)
