"""Token-budget micro-batching (host logic, no GPU): the oracle's restatement of the reference against
outputs of the reference's own module (tests/golden/reference_partition_vectors.json: the reference
holds no vectors for it, so its functions were run on seeded inputs, ties included), textbook results of
the largest differencing method, brute force and invariants; and the package's implementation against
the same vectors and against the oracle, partition for partition."""
import itertools
import json
import os
import random

import pytest
import torch

from mindspeed_rl_amd import seqlen_balancing as sb
from oracle import balancing as ob


def _sums(lengths, partitions):
    return sorted(sum(lengths[i] for i in p) for p in partitions)


def _is_partition(n, partitions):
    flat = sorted(i for p in partitions for i in p)
    return flat == list(range(n))


def test_differencing_method_textbook_cases():
    # the worked example of the largest differencing method: {8,7,6,5,4} splits 16/14 two ways and
    # {8}, {4,7}, {5,6} three ways
    lengths = [8, 7, 6, 5, 4]
    assert _sums(lengths, ob.karmarkar_karp(lengths, 2, False)) == [14, 16]
    parts = ob.karmarkar_karp(lengths, 3, False)
    assert sorted(sorted(lengths[i] for i in p) for p in parts) == [[4, 7], [5, 6], [8]]
    # two items, two bins; one bin; as many bins as items
    assert _sums([3, 9], ob.karmarkar_karp([3, 9], 2, False)) == [3, 9]
    assert ob.karmarkar_karp([5, 1, 2], 1, False) == [[1, 2, 0]] or _is_partition(3, ob.karmarkar_karp([5, 1, 2], 1, False))
    assert _sums([4, 4, 4, 4], ob.karmarkar_karp([4, 4, 4, 4], 4, False)) == [4, 4, 4, 4]
    # equal-size mode: every bin gets n / k items; a remainder is an error
    parts = ob.karmarkar_karp([1, 2, 3, 4, 5, 6, 7, 8], 2, True)
    assert [len(p) for p in parts] == [4, 4] and _sums([1, 2, 3, 4, 5, 6, 7, 8], parts) == [18, 18]
    with pytest.raises(ValueError):
        ob.karmarkar_karp([1, 2, 3], 2, True)


def test_oracle_invariants_and_brute_force():
    rnd = random.Random(5)
    for _ in range(200):
        n = rnd.randint(1, 9)
        lengths = [rnd.randint(1, 30) for _ in range(n)]
        k = rnd.randint(1, n)
        kk = ob.karmarkar_karp(lengths, k, False)
        greedy = ob.heapq_partition(lengths, k, False)
        assert len(kk) == k and len(greedy) == k and _is_partition(n, kk) and _is_partition(n, greedy)
        # brute force: the optimum makespan over all k^n assignments
        best = min(max(sum(l for l, b in zip(lengths, assign) if b == g) for g in range(k))
                   for assign in itertools.product(range(k), repeat=n)) if k ** n <= 20000 else None
        if best is not None:
            # longest-processing-time greedy is within 4/3 - 1/(3k) of the optimum (Graham), and the
            # two-way differencing method never ends further apart than its largest item
            assert max(_sums(lengths, greedy)) <= (4 / 3 - 1 / (3 * k)) * best + 1e-9
            assert max(_sums(lengths, kk)) >= best
            if k == 2:
                s = _sums(lengths, kk)
                assert s[1] - s[0] <= max(lengths)
        cap = max(lengths) + rnd.randint(0, 40)
        capped = ob.heapq_partition_with_max(lengths, k, cap)
        assert _is_partition(n, capped) and all(sum(lengths[i] for i in p) <= cap for p in capped)
        micro = ob.rearrange_micro_batches(lengths, cap, dynamic_max_batch_size=3)
        assert _is_partition(n, micro)
        assert len(micro) >= max(-(-sum(lengths) // cap), -(-n // 3))
    balanced = ob.get_seqlen_balanced_partitions([7, 1, 5, 3, 8, 2], 3, True)
    assert all(p == sorted(p) and len(p) == 2 for p in balanced) and _is_partition(6, balanced)
    with pytest.raises(ValueError):
        ob.get_seqlen_balanced_partitions([1, 2], 3, False)
    perm = [3, 0, 2, 1]
    inverse = ob.get_reverse_idx(perm)
    assert [perm[i] for i in inverse] == [0, 1, 2, 3] and [inverse[p] for p in perm] == [0, 1, 2, 3]


def test_package_matches_oracle_partition_for_partition():
    rnd = random.Random(9)
    for trial in range(400):
        n = rnd.randint(1, 70)
        # every third trial draws from four values only: many ties, which the tie-breaking rules decide
        lengths = [rnd.choice([5, 5, 7, 9]) if trial % 3 == 0 else rnd.randint(1, 4096) for _ in range(n)]
        k = rnd.randint(1, n)
        assert sb.karmarkar_karp(lengths, k, False) == ob.karmarkar_karp(lengths, k, False)
        assert sb.heapq_partition(lengths, k, False) == ob.heapq_partition(lengths, k, False)
        if n % k == 0:
            assert sb.karmarkar_karp(lengths, k, True) == ob.karmarkar_karp(lengths, k, True)
            assert sb.heapq_partition(lengths, k, True) == ob.heapq_partition(lengths, k, True)
            assert sb.get_seqlen_balanced_partitions(lengths, k, True) == \
                ob.get_seqlen_balanced_partitions(lengths, k, True)
        cap = max(lengths) + rnd.randint(0, 8192)
        assert sb.heapq_partition_with_max(lengths, k, cap) == ob.heapq_partition_with_max(lengths, k, cap)
        for cap_batch in (None, 1, 4, 16):
            assert sb.rearrange_micro_batches(lengths, cap, cap_batch) == ob.rearrange_micro_batches(lengths, cap, cap_batch)
    perm = list(range(50))
    rnd.shuffle(perm)
    assert sb.get_reverse_idx(perm) == ob.get_reverse_idx(perm)
    with pytest.raises(ValueError):
        sb.karmarkar_karp([1, 2, 3], 2, True)
    with pytest.raises(ValueError):
        sb.get_seqlen_balanced_partitions([1, 2], 3, False)
    with pytest.raises(NotImplementedError):
        sb.rearrange_micro_batches([1, 2], 8, dp_group=object())


def test_split_batches_with_dynamic_bsz():
    gen = torch.Generator().manual_seed(4)
    n = 24
    batch = {"prompt_length": torch.randint(1, 200, (n, 1), generator=gen),
             "response_length": torch.randint(1, 900, (n, 1), generator=gen),
             "responses": torch.randint(0, 100, (n, 16), generator=gen),
             "ragged": [torch.full((i % 3 + 1,), i) for i in range(n)],
             "note": "kept out"}
    lengths = (batch["prompt_length"] + batch["response_length"]).view(-1).tolist()
    micro, partitions = sb.split_batches_with_dynamic_bsz(batch, 4096, 8)
    assert partitions == ob.rearrange_micro_batches(lengths, 4096, 8)
    assert len(micro) == len(partitions)
    for mb, part in zip(micro, partitions):
        assert torch.equal(mb["responses"], batch["responses"][part])
        assert torch.equal(mb["ragged"], torch.cat([batch["ragged"][p] for p in part]))
        assert "note" not in mb
        assert int((mb["prompt_length"] + mb["response_length"]).sum()) <= 4096 or len(part) == 1
    order = [i for part in partitions for i in part]
    back = sb.get_reverse_idx(order)
    assert [order[j] for j in back] == list(range(n))


def _plain_best_fit_decreasing(lengths, cap):
    """Textbook best fit decreasing (no balancing pass): bin loads."""
    loads = []
    for length in sorted(lengths, reverse=True):
        fits = [b for b, load in enumerate(loads) if cap - load >= length]
        if fits:
            loads[min(fits, key=lambda b: cap - loads[b])] += length
        else:
            loads.append(length)
    return loads


def test_oracle_bin_packing_textbook_brute_force_and_invariants():
    # a worked best-fit-decreasing example: 8 | 4 4 | 2 joins the 8 (tightest fit, first on ties) | 1 1 -> 10 / 10
    parts = ob.balanced_bin_packing([4, 8, 1, 4, 2, 1], 10)
    assert _sums([4, 8, 1, 4, 2, 1], parts) == [10, 10] and _is_partition(6, parts)
    assert ob.balanced_bin_packing([], 10) == []
    assert ob.balanced_bin_packing([7], 7) == [[0]]
    with pytest.raises(ValueError):
        ob.balanced_bin_packing([3, 11], 10)
    # the balancing pass: best fit alone gives 9 / 2 at capacity 10; moving the 3 leaves 6 / 5
    assert _sums([6, 3, 2], ob.balanced_bin_packing([6, 3, 2], 10)) == [5, 6]
    rnd = random.Random(11)
    for _ in range(300):
        n = rnd.randint(1, 8)
        cap = rnd.randint(5, 40)
        lengths = [rnd.randint(1, cap) for _ in range(n)]
        parts = ob.balanced_bin_packing(lengths, cap)
        loads = [sum(lengths[i] for i in p) for p in parts]
        assert _is_partition(n, parts) and all(p for p in parts) and max(loads) <= cap
        plain = _plain_best_fit_decreasing(lengths, cap)
        # the balancing pass keeps the bin count and never widens the range of loads
        assert len(loads) == len(plain)
        assert max(loads) <= max(plain) and min(loads) >= min(plain)
        # bin count against the optimum (all assignments of n items to at most n bins): best fit
        # decreasing needs at most 11/9 OPT + 6/9 bins
        if n > 6:
            continue
        best = None
        for assign in itertools.product(range(n), repeat=n):
            used = {}
            for length, b in zip(lengths, assign):
                used[b] = used.get(b, 0) + length
            if max(used.values()) <= cap and (best is None or len(used) < best):
                best = len(used)
            if best == -(-sum(lengths) // cap):
                break
        assert len(loads) <= 11 * best / 9 + 6 / 9 + 1e-9


def test_bin_packing_matches_oracle():
    rnd = random.Random(17)
    for _ in range(400):
        n = rnd.randint(0, 40)
        cap = rnd.randint(8, 4096)
        lengths = [rnd.randint(1, cap) if rnd.random() < 0.3 else rnd.randint(1, max(1, cap // 4)) for _ in range(n)]
        want = ob.balanced_bin_packing(list(lengths), cap)
        assert sb.balanced_bin_packing(lengths, cap) == want
        assert sb.rearrange_micro_batches(lengths, cap, multimodal=True) == want
        assert ob.rearrange_micro_batches(lengths, cap, multimodal=True) == want
    # many equal lengths (ties everywhere) and a case the balancing pass changes three times
    for lengths, cap in (([5] * 13, 12), ([9, 9, 9, 1, 1, 1, 1, 1, 1], 12), ([10, 6, 5, 4, 3, 2, 2, 1], 11)):
        assert sb.balanced_bin_packing(lengths, cap) == ob.balanced_bin_packing(lengths, cap)
    with pytest.raises(ValueError, match="exceeds max_capacity"):
        sb.balanced_bin_packing([3, 11], 10)


def _plain(x):
    return [_plain(v) for v in x] if isinstance(x, (list, tuple)) else int(x)


def _call(mod, case, flag_by_env):
    fn = case["fn"]
    if fn in ("karmarkar_karp", "heapq_partition", "get_seqlen_balanced_partitions"):
        return getattr(mod, fn)(list(case["seqlen_list"]), case["k_partitions"], case["equal_size"])
    if fn == "heapq_partition_with_max":
        return mod.heapq_partition_with_max(list(case["seqlen_list"]), case["k_partitions"], case["max_token_len"])
    if fn == "balanced_bin_packing":
        return mod.balanced_bin_packing(list(case["seqlen_list"]), case["max_capacity"])
    if fn == "get_reverse_idx":
        return mod.get_reverse_idx(list(case["idx_map"]))
    assert fn == "rearrange_micro_batches"
    if flag_by_env:
        # the reference's own switch: is_multimodal() reads the process environment
        os.environ["IS_MULTIMODAL"] = "1" if case["multimodal"] else "0"
        try:
            return mod.rearrange_micro_batches(list(case["seqlen_list"]), case["max_token_len"], case["dynamic_max_batch_size"])
        finally:
            os.environ.pop("IS_MULTIMODAL", None)
    return mod.rearrange_micro_batches(list(case["seqlen_list"]), case["max_token_len"], case["dynamic_max_batch_size"],
                                       multimodal=case["multimodal"])


@pytest.mark.parametrize("which", ["oracle", "package"])
def test_partitioners_equal_the_reference_outputs(which):
    """Every partitioner, partition for partition and index for index, against what the reference's module
    returned for the same arguments: lists with few distinct lengths (nearly every comparison a tie), all
    lengths equal, response-like lengths and multiples of 128; 1 to 64 items, 1 to n groups, equal-size
    and free, budgets from the longest item to the whole batch, with and without a minimum number of
    micro-batches, and the capacity-bound packing of the multimodal branch."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_partition_vectors.json")
    with open(path) as fh:
        cases = json.load(fh)["cases"]
    assert len(cases) > 1000 and {c["fn"] for c in cases} == {
        "karmarkar_karp", "heapq_partition", "get_seqlen_balanced_partitions", "heapq_partition_with_max",
        "balanced_bin_packing", "rearrange_micro_batches", "get_reverse_idx"}
    mod, by_env = (ob, False) if which == "oracle" else (sb, True)
    for case in cases:
        got = _plain(_call(mod, case, by_env))
        assert got == case["out"], {k: v for k, v in case.items() if k != "out"}
