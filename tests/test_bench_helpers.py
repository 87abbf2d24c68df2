"""The bookkeeping of bench.py that needs no GPU: the byte count behind
`roofline.achieved`, the whole-batch comparison with the oracle, the source
hash that ties counter figures to a build."""
import json
import os

import numpy as np

import bench


def test_algorithmic_bytes_formula():
    # 4-byte ids and floats: query + entries + per expansion 8 + per adjacency
    # entry 4 + per distance (4 + 4 dp) + per result slot 8
    counters = [10, 640, 100, 50, 256]         # E, A, C, admitted, R
    B, dp, n_init = 2, 128, 64
    want = B * (4 * dp + n_init * 8) + 10 * 8 + 640 * 4 + 100 * (4 + 4 * dp) + 256 * 8
    assert bench.algorithmic_bytes(counters, B, dp, n_init) == want


def test_compare_search_tells_ties_from_mismatches():
    D = np.array([[1.0, 2.0, 2.0, 3.0], [1.0, 2.0, 3.0, 4.0]], np.float32)
    I = np.array([[5, 6, 7, 8], [1, 2, 3, 4]])
    same = bench.compare_search(I, D, I.copy(), D.copy())
    assert same == dict(distances_identical=True, rows_with_other_order_inside_ties=0,
                        rows_with_another_member_of_a_tie=0, rows_with_id_mismatch=0)
    # the two ids of a tie the other way round
    swapped = I.copy()
    swapped[0, 1], swapped[0, 2] = 7, 6
    r = bench.compare_search(I, D, swapped, D.copy())
    assert r['rows_with_other_order_inside_ties'] == 1 and r['rows_with_id_mismatch'] == 0
    # another node at exactly the same distance in the last place
    other = I.copy()
    other[1, 3] = 99
    r = bench.compare_search(I, D, other, D.copy())
    assert r['rows_with_another_member_of_a_tie'] == 1 and r['rows_with_id_mismatch'] == 0
    assert r['example']['row'] == 1 and r['example']['ids_b'] == [99]
    # a different distance is a mismatch
    D2 = D.copy()
    D2[1, 3] = 5.0
    r = bench.compare_search(I, D, other, D2)
    assert not r['distances_identical'] and r['rows_with_id_mismatch'] == 1


def test_traffic_figures_name_the_sources_they_were_measured_with():
    path = os.path.join(os.path.dirname(bench.__file__), 'profiles', 'traffic.json')
    entries = json.load(open(path))
    assert len(bench.kernel_sources_sha16()) == 16
    for key, entry in entries.items():
        assert entry['hbm_bytes_per_launch'] > 0 and len(entry['kernel_sources_sha16']) == 16
    value, fresh = bench.measured_traffic('c3/n=1000000/queries=10000/ef=32/spectrum_exponent=0.0')
    assert value == entries['c3/n=1000000/queries=10000/ef=32/spectrum_exponent=0.0']['hbm_bytes_per_launch']
    assert fresh in (True, False)
    assert bench.measured_traffic('no such workload') == (None, None)
    cfg = dict(bench.CONFIGS['c3'], name='c3')
    assert bench.traffic_key(cfg, 10000, 32) in entries


def test_the_parity_check_of_the_gpu_tests_tolerates_ties_only():
    """tests/common.py:assert_same_search — what the GPU parity tests pass or
    fail on: another order inside a tie passes, another id does not, another
    member of a tie passes only at the worst kept distance and only through
    the caller's check of those ids."""
    import pytest
    from common import assert_same_search
    D = np.array([[1.0, 2.0, 2.0, 3.0, 3.0]], np.float32)
    I = np.array([[5, 6, 7, 8, 9]])
    swapped = np.array([[5, 7, 6, 9, 8]])
    assert_same_search(I, D, swapped, D.copy())
    other = np.array([[5, 6, 7, 8, 4]])
    with pytest.raises(AssertionError, match='outside a tie'):
        assert_same_search(other, D, I, D.copy())
    asked = []
    assert_same_search(other, D, I, D.copy(),
                       worst_tie=lambda row, ids, dist: asked.append((row, sorted(ids), dist)))
    assert asked == [(0, [4, 8], 3.0)]
    # not at the worst distance: never tolerated
    inner = np.array([[5, 6, 4, 8, 9]])
    with pytest.raises(AssertionError, match='outside a tie'):
        assert_same_search(inner, D, I, D.copy(), worst_tie=lambda *a: None)
    with pytest.raises(AssertionError, match='distances differ'):
        assert_same_search(I, D, I, D + 1)
