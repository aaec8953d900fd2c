"""The planner's default against measurement, off the shapes its constants were calibrated on.

For seeded random products the autotuner times every macro-tile x split-K x tail-split candidate
(and the streaming or short-K kernel where one applies); the default choice has to be within 30 %
of the fastest candidate for all of them.  How many are within 10 % (85 % of the shapes and more on
the devices this was developed on) and the worst ratios are printed, so a run shows where the model
is weakest; that share is not asserted, since timings of 10 to 100 microseconds move by several
percent from launch to launch and more from device to device."""
import numpy as np
import pytest

import cake_on_cpu_amd as cake

pytestmark = pytest.mark.gpu


def _shapes(seed, count):
    rng = np.random.default_rng(seed)

    def dim(lo, hi):
        v = int(round(2 ** rng.uniform(np.log2(lo), np.log2(hi))))
        return v if rng.random() < 0.5 else max(4, v // 4 * 4)

    out = []
    while len(out) < count:
        M, N, K = dim(33, 8192), dim(33, 8192), dim(16, 8192)
        if 2e8 <= 2.0 * M * N * K <= 2.5e11:
            out.append((M, N, K))
    return out


def test_default_plan_is_close_to_the_measured_best():
    shapes = _shapes(31, 28)
    ratios = []
    try:
        for (M, N, K) in shapes:
            cake.tune_clear()
            d = cake.plan(M, N, K)
            p, best, base = cake.autotune(M, N, K, budget_seconds=0.6)
            assert best > 0 and base >= best
            ratios.append((base / best, (M, N, K), d.as_dict(), p.as_dict()))
            print(f"planner M={M} N={N} K={K}: default {base * 1e6:.1f} us, best {best * 1e6:.1f} us, ratio {base / best:.3f}",
                  flush=True)
    finally:
        cake.tune_clear()
    ratios.sort(key=lambda r: -r[0])
    for r, shape, d, p in ratios[:5]:
        print(f"  weakest: {shape} ratio {r:.3f}: default {d['tile_m']}x{d['tile_n']}x{d['tile_k']} split {d['split_k']} "
              f"tail {d['tail_tiles']} kernel {d['kernel']}; best {p['tile_m']}x{p['tile_n']}x{p['tile_k']} split {p['split_k']} "
              f"tail {p['tail_tiles']}", flush=True)
    within = sum(r[0] <= 1.10 for r in ratios)
    print(f"planner: default within 10 % of the measured best on {within} of {len(ratios)} shapes", flush=True)
    assert ratios[0][0] <= 1.30, ratios[0]
