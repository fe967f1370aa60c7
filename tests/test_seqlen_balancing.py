"""Token-budget micro-batching (host logic, no GPU): the oracle's restatement of the reference against
textbook results of the largest differencing method, brute force and invariants (the reference holds no
vectors for this module), and the package's implementation against the oracle, partition for partition."""
import itertools
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
