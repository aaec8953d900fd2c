"""The autotuner on the device: it measures explicit tile / split-K / tail-split
choices, keeps the fastest per product, and the products computed through a
tuned plan stay within the parity bar."""
import numpy as np
import pytest

import cake_on_cpu_amd as cake
import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _clean_table():
    cake.tune_clear()
    yield
    cake.tune_clear()


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (300, 5000, 260), (2111, 200, 2111), (4352, 512, 1024)],
                         ids=lambda s: "x".join(map(str, s)))
def test_autotune_picks_a_measured_plan_and_results_stay_right(shape, tmp_path):
    M, K, N = shape
    before = cake.plan(M, N, K).as_dict()
    print(f"autotune M={M} K={K} N={N} default={before}", flush=True)
    plan, best, base = cake.autotune(M, N, K, budget_seconds=3.0)
    print(f"  tuned={plan.as_dict()} best={best * 1e6:.1f} us default={base * 1e6:.1f} us", flush=True)
    assert best > 0 and base > 0 and best <= base          # the default is one of the candidates
    assert cake.tune_count() >= 1
    now = cake.plan(M, N, K).as_dict()
    assert now == plan.as_dict()                            # later plans use the measured choice
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    Cm = np.zeros((M, N), np.float32)
    cake.cake_sgemm(A, B, Cm, M, N, K, 4)
    C64, S = oracle.gemm_f64(A, B)
    assert oracle.max_rel_err(Cm, C64, S) <= 5e-6
    # the table survives a save / clear / load cycle and gives the same plan
    path = tmp_path / "t.txt"
    cake.tune_save(path)
    cake.tune_clear()
    assert cake.plan(M, N, K).as_dict() == before
    assert cake.tune_load(path) >= 1
    assert cake.plan(M, N, K).as_dict() == now


@pytest.mark.parametrize("shape", [(16, 2048, 4096), (4096, 1024, 8), (4096, 64, 4096), (2000, 48, 3000), (2111, 96, 2111)],
                         ids=lambda s: "x".join(map(str, s)))
def test_autotune_of_a_streaming_shape(shape):
    """Few rows or columns, or a short K under many tiles: the kernel those shapes have of their own
    is the measured default, a tile only enters the table when it is faster, and the product stays
    right either way."""
    M, K, N = shape
    plan, best, base = cake.autotune(M, N, K, budget_seconds=2.0)
    print(f"autotune streaming M={M} K={K} N={N} best={best * 1e6:.1f} us default={base * 1e6:.1f} us "
          f"entries={cake.tune_count()}", flush=True)
    assert best > 0 and base > 0 and best <= base
    assert (cake.tune_count() >= 1) == (best < base)       # no entry when the streaming kernel wins
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    Cm = np.zeros((M, N), np.float32)
    cake.cake_sgemm(A, B, Cm, M, N, K, 4)
    C64, S = oracle.gemm_f64(A, B)
    assert oracle.max_rel_err(Cm, C64, S) <= 5e-6
