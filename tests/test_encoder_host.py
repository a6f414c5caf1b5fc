"""Host-side logic of the encoder builder that needs no GPU."""
import numpy as np

from tensorrt_amd.encoder import split_runs


def _cu(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def test_split_runs_balances_tokens_on_sequence_boundaries():
    lens = np.random.default_rng(1).integers(128, 385, 128)
    cu = _cu(lens)
    runs = split_runs(cu, 2)
    assert runs[0][0] == 0 and runs[-1][1] == 128 and runs[0][1] == runs[1][0]
    a, b = (int(cu[hi] - cu[lo]) for lo, hi in runs)
    assert abs(a - b) <= int(lens.max())          # within one sequence of the middle
    three = split_runs(cu, 3)
    assert [r[0] for r in three[1:]] == [r[1] for r in three[:-1]] and len(three) == 3
    sizes = [int(cu[hi] - cu[lo]) for lo, hi in three]
    assert max(sizes) - min(sizes) <= 2 * int(lens.max())


def test_split_runs_degenerate_batches():
    assert split_runs(_cu([77]), 2) == [(0, 1)]                 # one sequence cannot be cut
    assert split_runs(_cu([5, 9]), 4) == [(0, 1), (1, 2)]       # never more runs than sequences
    assert split_runs(_cu([0, 0, 150, 40]), 2) == [(0, 3), (3, 4)]
    assert split_runs(_cu([90, 60, 0, 0]), 2) == [(0, 1), (1, 4)]
    assert split_runs(_cu([0, 0, 0, 12]), 2) == [(1, 4)]        # a run of empty sequences is left out
    assert split_runs(_cu([0, 0]), 2) == []                     # nothing to compute
    whole = split_runs(_cu([3, 4, 5]), 1)
    assert whole == [(0, 3)]
