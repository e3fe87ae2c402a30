"""The CPU oracle against every vector the reference's own tests hold for the path."""
import numpy as np
import pytest

import golden_cases as gc

CASES = gc.load_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["name"][:50] for c in CASES])
def test_oracle_matches_reference_vector(orc, case):
    gc.run_case(orc, case)


def test_threaded_oracle_is_bit_identical_to_single_thread(orc):
    from sliced_amd import rng
    rows, cols = 300, 5000
    x = rng.uniform(rows * cols, -10, 10, tag=0)
    g = rng.normal(rows * cols, 1.0, tag=1)

    def run():
        s = orc.softmax(rows, cols, x)
        return [orc.sum_rows(cols, x), orc.sum_cols(cols, x), orc.max_rows(cols, x), orc.max_cols(cols, x),
                s, orc.softmax_grad(rows, cols, s, g), orc.transpose(rows, cols, x),
                orc.gemm(rows, 200, cols, x, x[:cols * 200]), orc.Tgemm(cols, 64, rows, x, g[:rows * 64]),
                orc.gemmT(rows, 32, cols, x, g[:32 * cols])]

    orc.set_threads(1)
    a = run()
    orc.set_threads(min(8, orc.max_threads()))
    b = run()
    for u, v in zip(a, b):
        assert np.array_equal(u, v)
