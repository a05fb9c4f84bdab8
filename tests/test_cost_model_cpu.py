"""The fused call's choice of kernel family against measured times (host logic only: ssd_query_fused_plan touches no
device).  The reference has one kernel per fused wrapper (kernels/fused_globalbar.py:201-266,
kernels/fused_concurrent.py:255-331) and no such choice; here four families compute the same result and the library
ranks them by an estimate of their duration (csrc/ssd_cost.h).

The tables hold microseconds per call on one MI355X at steady clocks (300 ms of the same call before each timing,
bf16 inputs, fp32 passed states, random data): the chain kernel forced with 4 / 2 / 1 chunks per item, the call without
a workspace (what ssd_fused_chunk_state_passing_fwd runs), and the four-tile and token-split kernels forced through
ssd_set_token_split (the dispatcher reaches those two only where the call without a workspace picks them).  FITTED
is the sweep the estimates were fitted on; HELD_OUT was measured afterwards, on shapes the fit had not seen, with the
dispatcher as it is now."""
import pytest

import ssd_amd as ops

# batch, seqlen, nheads, headdim, dstate, ngroups, chunk, packed sequences,  chain R=4, R=2, R=1, no workspace, four-tile, token-split
FITTED = [
    (1, 2048, 80, 64, 128, 1, 256, 0,  39.3, 32.5, 38.5, 23.3, 44.9, 23.2),
    (1, 4096, 80, 64, 128, 1, 256, 0,  47.3, 44.0, 52.4, 41.5, 82.9, 41.4),
    (1, 8192, 80, 64, 128, 1, 256, 0,  71.6, 63.0, 86.6, 77.9, 158.9, 77.5),
    (1, 16384, 80, 64, 128, 1, 256, 0,  116.3, 127.3, 213.2, 142.9, 327.5, 207.7),
    (2, 2048, 80, 64, 128, 1, 256, 0,  41.1, 41.2, 41.3, 34.6, 45.1, 34.5),
    (2, 4096, 80, 64, 128, 1, 256, 0,  66.8, 57.7, 64.7, 63.4, 83.2, 62.8),
    (2, 8192, 80, 64, 128, 1, 256, 0,  107.3, 104.0, 135.1, 134.7, 179.8, 182.4),
    (2, 16384, 80, 64, 128, 1, 256, 0,  185.0, 196.5, 301.1, 274.7, 354.8, 363.0),
    (4, 2048, 80, 64, 128, 1, 256, 0,  67.3, 55.1, 57.4, 46.5, 46.4, 49.6),
    (4, 4096, 80, 64, 128, 1, 256, 0,  103.1, 97.8, 109.7, 112.3, 111.6, 135.4),
    (4, 8192, 80, 64, 128, 1, 256, 0,  175.1, 176.6, 198.3, 210.7, 211.1, 262.3),
    (4, 16384, 80, 64, 128, 1, 256, 0,  326.1, 330.0, 379.6, 418.5, 418.3, 519.3),
    (8, 2048, 80, 64, 128, 1, 256, 0,  104.0, 94.8, 106.3, 113.5, 113.8, 127.5),
    (8, 4096, 80, 64, 128, 1, 256, 0,  172.7, 174.3, 189.1, 216.2, 216.7, 240.5),
    (8, 8192, 80, 64, 128, 1, 256, 0,  328.6, 330.7, 365.0, 422.3, 422.5, 470.3),
    (8, 16384, 80, 64, 128, 1, 256, 0,  635.6, 646.3, 687.3, 839.0, 839.7, 932.8),
    (4, 4096, 24, 64, 128, 1, 256, 0,  47.3, 45.7, 52.9, 41.3, 82.8, 41.3),
    (4, 8192, 24, 64, 128, 1, 256, 0,  74.2, 67.3, 93.2, 77.1, 158.8, 77.2),
    (8, 2048, 24, 64, 128, 1, 256, 0,  41.6, 42.5, 43.9, 33.9, 45.8, 34.0),
    (4, 4096, 48, 64, 128, 1, 256, 0,  70.8, 61.5, 70.3, 61.6, 83.2, 61.7),
    (4, 8192, 48, 64, 128, 1, 256, 0,  114.9, 121.1, 162.8, 155.9, 182.1, 186.3),
    (8, 2048, 48, 64, 128, 1, 256, 0,  67.8, 58.5, 62.9, 46.8, 47.7, 52.2),
    (4, 4096, 128, 64, 128, 1, 256, 0,  142.3, 144.4, 155.3, 117.8, 115.1, 185.6),
    (4, 8192, 128, 64, 128, 1, 256, 0,  261.6, 265.3, 285.3, 224.1, 225.5, 363.2),
    (8, 2048, 128, 64, 128, 1, 256, 0,  149.0, 151.5, 156.8, 135.4, 135.7, 189.0),
    (4, 8192, 80, 64, 64, 1, 256, 0,  124.9, 130.8, 146.2, 166.6, 167.7, 193.8),
    (4, 8192, 80, 64, 128, 1, 128, 0,  255.4, 272.5, 353.8, 280.7, 280.9, 398.6),
    (4, 8192, 40, 128, 128, 1, 256, 0,  174.6, 174.0, 198.2, 211.3, 211.2, 261.4),
    (4, 8192, 128, 64, 128, 8, 256, 0,  267.3, 269.3, 296.3, 229.7, 232.0, 360.5),
    (1, 65536, 128, 64, 128, 8, 256, 0,  542.6, 655.6, 1134.1, 871.7, 1308.5, 861.9),
    (1, 32768, 80, 64, 128, 1, 256, 0,  218.5, 287.2, 516.5, 301.2, 649.3, 412.5),
    (1, 32768, 80, 64, 128, 1, 256, 16,  198.8, 269.2, 466.5, 312.7, 719.7, 421.6),
    (2, 16384, 80, 64, 128, 1, 256, 6,  184.9, 200.2, 283.7, 279.4, 378.6, 366.9),
    (16, 1024, 80, 64, 128, 1, 256, 0,  103.8, 95.7, 107.8, 98.2, 98.1, 130.0),
    (32, 512, 80, 64, 128, 1, 256, 0,  100.2, 98.3, 109.9, 100.1, 100.0, 141.5),
]
HELD_OUT = [
    (3, 6144, 64, 64, 128, 1, 256, 0,  100.1, 95.1, 107.3, 110.7, 133.5, 136.7),
    (2, 12288, 96, 64, 128, 1, 256, 0,  168.7, 169.1, 224.7, 244.8, 271.4, 276.4),
    (6, 3072, 32, 64, 128, 1, 256, 0,  65.2, 55.0, 58.4, 47.5, 64.4, 47.5),
    (1, 24576, 48, 64, 128, 1, 256, 0,  126.3, 150.3, 260.0, 131.2, 479.2, 284.8),
    (5, 2560, 80, 64, 128, 1, 256, 0,  87.1, 80.3, 86.0, 78.1, 77.6, 103.2),
    (2, 4096, 128, 64, 64, 1, 256, 0,  55.3, 57.0, 66.1, 66.0, 65.9, 46.2),
    (4, 8192, 64, 64, 128, 1, 128, 0,  206.7, 227.0, 329.1, 252.8, 252.7, 277.0),
    (1, 131072, 32, 64, 128, 1, 256, 0,  502.8, 715.5, 1514.3, 647.8, 2508.3, 1465.1),
    (12, 1536, 40, 64, 128, 1, 256, 0,  58.6, 57.4, 61.7, 39.5, 40.6, 49.7),
    (1, 8192, 256, 64, 128, 1, 256, 0,  141.9, 142.1, 176.4, 179.0, 179.6, 189.4),
    (3, 4096, 80, 64, 128, 1, 256, 0,  74.1, 79.3, 85.3, 91.4, 94.6, 91.5),
    (6, 8192, 80, 64, 128, 1, 256, 0,  254.5, 252.9, 275.2, 243.7, 243.8, 368.2),
    (2, 2048, 128, 64, 128, 8, 256, 0,  44.3, 45.7, 52.1, 46.3, 46.5, 34.9),
    (1, 16384, 24, 64, 128, 1, 256, 0,  90.6, 95.8, 151.6, 144.8, 308.8, 144.8),
    (10, 2048, 64, 64, 128, 1, 256, 0,  105.1, 93.3, 102.6, 109.2, 108.5, 120.5),
    (2, 32768, 32, 64, 128, 1, 256, 12,  175.6, 243.0, 433.9, 257.5, 717.2, 399.0),
    (7, 4096, 48, 64, 128, 1, 256, 0,  105.5, 104.9, 114.1, 107.0, 106.8, 134.6),
    (1, 4096, 128, 128, 128, 1, 256, 0,  75.4, 79.7, 86.9, 90.8, 90.7, 82.8),
]


def _picked_and_best(row):
    b, L, H, P, N, G, Q, _, r4, r2, r1, no_ws, _, _ = row
    plan = ops.fused_plan(b, L, H, P, N, G, Q, workspace=True, compute_units=256)
    reachable = {4: r4, 2: r2, 1: r1, 0: no_ws}        # what the dispatcher can pick with a workspace
    picked = reachable[plan["chunks_per_item"] if plan["family"] == "chain" else 0]
    return plan, picked, min(reachable.values())


@pytest.mark.parametrize("table, worst, mean", [(FITTED, 1.04, 1.005), (HELD_OUT, 1.06, 1.015)], ids=["fitted", "held-out"])
def test_the_family_picked_is_close_to_the_best_one_measured(table, worst, mean):
    ratios = []
    for row in table:
        plan, picked, best = _picked_and_best(row)
        assert picked <= worst * best, (row[:8], plan, picked, best)
        ratios.append(picked / best)
    assert sum(ratios) / len(ratios) <= mean


def test_estimates_are_within_a_quarter_of_the_measurement_where_a_family_is_picked():
    for row in FITTED + HELD_OUT:
        plan, picked, _ = _picked_and_best(row)
        est = plan["estimate_us"][plan["family"]]
        assert 0.75 * picked <= est <= 1.25 * picked, (row[:8], plan, picked)


def test_the_benchmark_configurations_keep_their_kernels():
    # b=4 L=8192 H=80, the packed b=1 L=32768 H=80 and the grouped b=1 L=131072 H=128: chain kernel, four chunks per item;
    # b=8 L=2048 H=24: token-split
    for b, L, H, G in ((4, 8192, 80, 1), (1, 32768, 80, 1), (1, 131072, 128, 8)):
        plan = ops.fused_plan(b, L, H, 64, 128, G, 256)
        assert (plan["family"], plan["chunks_per_item"]) == ("chain", 4), plan
    assert ops.fused_plan(8, 2048, 24, 64, 128, 1, 256)["family"] == "token_split"


def test_without_a_workspace_the_chain_kernel_is_never_planned():
    for row in FITTED + HELD_OUT:
        plan = ops.fused_plan(*row[:7], workspace=False)
        assert plan["family"] != "chain" and plan["chunks_per_item"] == 0


def test_other_compute_unit_counts_rescale_the_choice():
    # half the device at half the batch is the same problem per compute unit
    full = ops.fused_plan(4, 8192, 80, 64, 128, 1, 256, compute_units=256)
    half = ops.fused_plan(2, 8192, 80, 64, 128, 1, 256, compute_units=128)
    assert (full["family"], full["chunks_per_item"]) == (half["family"], half["chunks_per_item"])
    assert abs(full["estimate_us"]["chain"] - half["estimate_us"]["chain"]) < 1e-3


def test_sizes_the_fast_kernels_do_not_cover_fall_to_the_generic_family():
    plan = ops.fused_plan(1, 1000, 6, 48, 40, 1, 100)
    assert plan["family"] == "generic" and plan["estimate_us"]["chain"] is None
    with pytest.raises(Exception):
        ops.fused_plan(1, 1024, 7, 64, 128, 2, 256)          # nheads % ngroups
