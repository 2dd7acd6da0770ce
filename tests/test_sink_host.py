"""Host logic of the ``kivi_sink`` cache, pinned against brute force on small random cases: the
running top-k by (norm descending, position ascending) and the stand-in search
(veloxquant_mlx/cache/sink_cache.py:87-112, 152-173)."""

import random

import torch

from veloxquant_mlx_amd.cache.sink_cache import _TopNorms, _stand_in_index


def _brute_top(history, n):
    """history: list of (pos, norm) in arrival order -> positions of the n largest, ties to the lower position."""
    return [p for p, _ in sorted(history, key=lambda pv: (-pv[1], pv[0]))[:n]]


def test_running_top_norms_match_brute_force_with_ties():
    rng = random.Random(5)
    for n in (1, 3, 5):
        top = _TopNorms(n)
        hist = [[], []]
        pos = 0
        for step in range(12):
            S = rng.choice([1, 1, 4, 9])
            # few distinct values: ties are the rule
            norms = torch.tensor([[float(rng.randint(0, 4)) for _ in range(S)] for _ in range(2)])
            top.fold(norms, pos)
            for b in range(2):
                hist[b] += [(pos + i, float(norms[b, i])) for i in range(S)]
            pos += S
            for b in range(2):
                # the running prune keeps what the top-n of the whole history is: a candidate that
                # lost its place can only have lost it to n better ones, which stay better
                assert top.positions(b) == _brute_top(hist[b], n), (n, step, b)
        top.drop_from(pos - 7)
        for b in range(2):
            kept = [pv for pv in hist[b] if pv[0] < pos - 7]
            assert set(top.positions(b)) <= {p for p, _ in kept}
            assert top.positions(b) == [p for p in _brute_top(hist[b], n) if p < pos - 7]
    assert _TopNorms(0).positions(0) == []


def _brute_stand_in(mask):
    n = len(mask)
    out = list(range(n))
    for i in range(n):
        if not mask[i]:
            continue
        below = [j for j in range(i - 1, -1, -1) if not mask[j]]
        above = [j for j in range(i + 1, n) if not mask[j]]
        out[i] = below[0] if below else (above[0] if above else i)
    return out


def test_stand_in_index_matches_search():
    rng = random.Random(9)
    cases = [[True] * 6, [False] * 6, [True, False, False, True, True], [False, True, True, True], [True, True, False]]
    cases += [[rng.random() < 0.4 for _ in range(rng.randint(1, 40))] for _ in range(50)]
    for mask in cases:
        got = _stand_in_index(torch.tensor([mask, mask[::-1]]))
        assert got[0].tolist() == _brute_stand_in(mask)
        assert got[1].tolist() == _brute_stand_in(mask[::-1])


def test_inside_marks_the_block_rows():
    top = _TopNorms(2)
    top.fold(torch.tensor([[1.0, 9.0, 2.0, 8.0], [7.0, 0.0, 0.5, 6.0]]), 10)
    assert top.positions(0) == [11, 13] and top.positions(1) == [10, 13]
    assert top.inside(10, 12).tolist() == [[False, True], [True, False]]
    assert top.inside(12, 14).tolist() == [[False, True], [False, True]]
