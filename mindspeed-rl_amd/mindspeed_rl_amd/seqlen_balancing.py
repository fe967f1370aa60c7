"""Token-budget micro-batching: which samples form each micro-batch of the loss path.

Host-side mirror of ``mindspeed_rl/utils/seqlen_balancing.py`` (``karmarkar_karp``,
``heapq_partition``, ``get_seqlen_balanced_partitions``, ``heapq_partition_with_max``,
``rearrange_micro_batches``, ``get_reverse_idx``) and of the splitting step of
``BaseTrainingEngine._split_batches_with_dynamic_bsz`` (``models/base/base_training_engine.py:
160-187``), with the reference's names, arguments, results (including its tie-breaking, so that
the same lengths give the same micro-batches) and errors.  This is pure host logic on a few
hundred integers; it decides the row count T of every sweep.  One data-parallel rank: the MAX
all-reduce of the bin count is not built.  The capacity-bound bin packing the reference uses for
multimodal batches (``balanced_bin_packing``, ``:191-307``) is selected by the reference's
process-wide switch (``is_multimodal()``, the environment variable IS_MULTIMODAL) or explicitly
with ``multimodal=True`` / ``False``.
"""
import heapq
from typing import Dict, List, Tuple

import torch

from .functional import is_multimodal


class _Reversed:
    """Inverts the order of the wrapped key inside a tuple comparison."""

    __slots__ = ("key",)

    def __init__(self, key):
        self.key = key

    def __lt__(self, other):
        return other.key < self.key

    def __eq__(self, other):
        return self.key == other.key


class _Bins:
    """k bins kept in descending order of (load, size, members); members are (index, length)."""

    __slots__ = ("loads", "members", "rank")

    def __init__(self, k, seed):
        self.loads = [0] * k
        self.members = [[] for _ in range(k)]
        for slot, (idx, length) in enumerate(seed):
            self.loads[slot] = length
            self.members[slot].append((idx, length))
        self._settle()

    def _bin_key(self, b):
        return (self.loads[b], len(self.members[b]), self.members[b])

    def _settle(self):
        order = sorted(range(len(self.loads)), key=self._bin_key, reverse=True)
        self.loads = [self.loads[b] for b in order]
        self.members = [self.members[b] for b in order]
        # popped first: the largest spread, then the largest heaviest bin
        self.rank = (self.loads[-1] - self.loads[0], _Reversed(self._bin_key(0)))

    def absorb(self, other):
        """Differencing step: the heaviest bin takes the other's lightest, and so on down."""
        k = len(self.loads)
        for b in range(k):
            src = k - 1 - b
            self.members[b].extend(other.members[src])
            self.loads[b] += other.loads[src]
        self._settle()

    def __lt__(self, other):
        return self.rank < other.rank


def karmarkar_karp(seqlen_list: List[int], k_partitions: int, equal_size: bool):
    """Largest differencing method for k partitions; returns k lists of item indices."""
    by_length = sorted((length, idx) for idx, length in enumerate(seqlen_list))
    if equal_size:
        if len(seqlen_list) % k_partitions != 0:
            raise ValueError(f"{len(seqlen_list)} % {k_partitions} != 0")
        seeds = [[(idx, length) for length, idx in by_length[lo:lo + k_partitions]]
                 for lo in range(0, len(by_length), k_partitions)]
    else:
        seeds = [[(idx, length)] for length, idx in by_length]
    heap = []
    for seed in seeds:
        heapq.heappush(heap, _Bins(k_partitions, seed))
    while len(heap) > 1:
        widest = heapq.heappop(heap)
        widest.absorb(heapq.heappop(heap))
        heapq.heappush(heap, widest)
    partitions = [[idx for idx, _ in members] for members in heap[0].members]
    if equal_size:
        for partition in partitions:
            if len(partition) * k_partitions != len(seqlen_list):
                raise ValueError(f"{len(partition)} * {k_partitions} != {len(seqlen_list)}")
    return partitions


def _longest_first(seqlen_list):
    return sorted(((length, idx) for idx, length in enumerate(seqlen_list)), reverse=True)


def heapq_partition(seqlen_list: List[int], k_partitions: int, equal_size: bool):
    """Longest item first onto the lightest group; with ``equal_size`` a group is closed once it
    holds its share of the items."""
    share = len(seqlen_list) // k_partitions
    open_groups = [[0, 0, g, []] for g in range(k_partitions)]      # load, size, id, members
    closed = []
    for length, idx in _longest_first(seqlen_list):
        load, size, gid, members = heapq.heappop(open_groups)
        members.append(idx)
        if equal_size and size + 1 >= share:
            closed.append(members)
        else:
            heapq.heappush(open_groups, [load + length, size + 1, gid, members])
    partitions = closed + [g[3] for g in open_groups]
    if equal_size:
        for i, partition in enumerate(partitions):
            if len(partition) * k_partitions != len(seqlen_list):
                raise ValueError(f"Partition {i} has {len(partition)} items, expected {share}")
    return partitions


def get_seqlen_balanced_partitions(seqlen_list: List[int], k_partitions: int, equal_size: bool):
    """k index lists with balanced length sums, each sorted ascending."""
    if k_partitions > len(seqlen_list):
        raise ValueError(f"number of items:[{len(seqlen_list)}] < k_partitions:[{k_partitions}]")
    return [sorted(p) for p in heapq_partition(seqlen_list, k_partitions, equal_size)]


def heapq_partition_with_max(seqlen_list: List[int], k_partitions: int, max_token_len: int):
    """Like :func:`heapq_partition`, but a group that the next item would push over
    ``max_token_len`` is closed and a new group is opened with that item."""
    open_groups = [[0, 0, g, []] for g in range(k_partitions)]
    next_id = k_partitions
    closed = []
    for length, idx in _longest_first(seqlen_list):
        lightest = heapq.heappop(open_groups)
        if lightest[0] + length > max_token_len:
            closed.append(lightest[3])
            heapq.heappush(open_groups, [length, 1, next_id, [idx]])
            next_id += 1
        else:
            lightest[0] += length
            lightest[1] += 1
            lightest[3].append(idx)
            heapq.heappush(open_groups, lightest)
    return closed + [g[3] for g in open_groups]


def balanced_bin_packing(seqlen_list: List[int], max_capacity: int):
    """Reference: ``utils/seqlen_balancing.py:191-307``.  Best fit decreasing under a hard capacity
    (longest item first into the fullest bin that still takes it, a new bin if none does), then at
    most three single-item moves from a fuller to an emptier bin that narrow their gap.  Returns
    the bins as index lists, in the order the balancing pass leaves them (ascending load at its
    last sort).  ``ValueError`` for an item longer than the capacity."""
    if not seqlen_list:
        return []
    loads: List[int] = []
    members: List[List[Tuple[int, int]]] = []
    for length, idx in _longest_first(seqlen_list):
        if length > max_capacity:
            raise ValueError(f"Item with seqlen {length} exceeds max_capacity {max_capacity}")
        room = [max_capacity - load for load in loads]
        fits = [b for b in range(len(loads)) if room[b] >= length]
        if fits:
            target = min(fits, key=lambda b: (room[b], b))
            loads[target] += length
            members[target].append((idx, length))
        else:
            loads.append(length)
            members.append([(idx, length)])
    for _ in range(3 if len(loads) > 1 else 0):
        order = sorted(range(len(loads)), key=lambda b: loads[b])          # stable, ascending load
        loads = [loads[b] for b in order]
        members = [members[b] for b in order]
        move = _first_narrowing_move(loads, members, max_capacity)
        if move is None:
            break
        heavy, light, slot = move
        item = members[heavy].pop(slot)
        members[light].append(item)
        loads[heavy] -= item[1]
        loads[light] += item[1]
    return [[idx for idx, _ in bin_members] for bin_members in members]


def _first_narrowing_move(loads, members, max_capacity):
    """(heavy bin, light bin, position in the heavy bin) of the first item, scanning the fullest
    bin first against the emptiest first, whose move keeps the capacity and narrows the gap."""
    for heavy in range(len(loads) - 1, 0, -1):
        for light in range(heavy):
            gap = loads[heavy] - loads[light]
            if gap <= 1:
                break
            for slot, (_, length) in enumerate(members[heavy]):
                if loads[light] + length <= max_capacity and abs(loads[heavy] - loads[light] - 2 * length) < gap:
                    return heavy, light, slot
    return None


def rearrange_micro_batches(seqlen_list: List[int], max_token_len: int, dynamic_max_batch_size: int = None,
                            dp_group=None, multimodal: bool = None):
    """Micro-batches (index lists) whose token sums are balanced: the bin count comes from the
    capped greedy pass (at least ``ceil(sum / max_token_len)``, and at least
    ``ceil(n / dynamic_max_batch_size)``), the assignment from the differencing method.  With
    ``multimodal`` the capacity-bound bin packing decides both (reference ``:356-359``)."""
    if multimodal is None:
        multimodal = is_multimodal()
    if multimodal:
        return balanced_bin_packing(seqlen_list, max_token_len)
    if dp_group is not None:
        raise NotImplementedError("the bin count is not synchronised across ranks on this path (one GPU)")
    floor_bins = (sum(seqlen_list) + max_token_len - 1) // max_token_len
    k_partitions = len(heapq_partition_with_max(seqlen_list, floor_bins, max_token_len))
    if dynamic_max_batch_size is not None:
        k_partitions = max(k_partitions, (len(seqlen_list) + dynamic_max_batch_size - 1) // dynamic_max_batch_size)
    return karmarkar_karp(seqlen_list, k_partitions, equal_size=False)


def get_reverse_idx(idx_map):
    """Inverse permutation: ``out[idx_map[i]] = i``."""
    reverse = list(idx_map)
    for position, idx in enumerate(idx_map):
        reverse[idx] = position
    return reverse


def split_batches_with_dynamic_bsz(batch: Dict, max_packing_token: int,
                                   dynamic_max_batch_size: int) -> Tuple[List[Dict], List[List[int]]]:
    """Reference: ``base_training_engine.py:160-187``.  The sequence lengths cross to the host in
    one copy (the reference calls ``.item()`` twice per sample); tensors are split by index lists,
    lists of tensors by concatenation."""
    lengths = (batch["prompt_length"].reshape(-1) + batch["response_length"].reshape(-1)).cpu().tolist()
    partitions = rearrange_micro_batches(lengths, max_packing_token, dynamic_max_batch_size=dynamic_max_batch_size)
    batches = [{} for _ in partitions]
    for key, value in batch.items():
        if isinstance(value, torch.Tensor):
            for micro, partition in zip(batches, partitions):
                micro[key] = value[partition]
        elif isinstance(value, list):
            for micro, partition in zip(batches, partitions):
                micro[key] = torch.concat([value[p] for p in partition])
    return batches, partitions
