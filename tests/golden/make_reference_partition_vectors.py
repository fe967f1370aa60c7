"""Writes tests/golden/reference_partition_vectors.json: inputs and outputs of the REFERENCE's own
micro-batch partitioners (``mindspeed_rl/utils/seqlen_balancing.py``), executed in the build container.

Why this module is run and not only read: the reference holds no test, fixture or example for these
functions, and what has to be pinned is their tie-breaking (which of two equal sums, spreads or
lengths comes first), which no closed form or invariant fixes.  Everything else on the path is pinned
without running the reference.

How: the one file is loaded by path.  Its only import from its own package is ``is_multimodal``
(``from mindspeed_rl.utils import is_multimodal``), and importing the package itself needs ray,
tensordict, torch_npu ...; so the two package names are pre-seeded in ``sys.modules`` with empty
modules whose single attribute ``is_multimodal`` returns what the case asks for.  No line of the
file is changed or copied; only its inputs and outputs are kept.  Run from the repository root:

    python tests/golden/make_reference_partition_vectors.py

It needs /root/reference (absent on the GPU box; the tests read the JSON only).
"""
import importlib.util
import json
import os
import random
import sys
import types

REFERENCE_FILE = "/root/reference/mindspeed_rl/utils/seqlen_balancing.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_partition_vectors.json")

_multimodal = [False]


def load_reference():
    pkg = types.ModuleType("mindspeed_rl")
    pkg.__path__ = []
    utils = types.ModuleType("mindspeed_rl.utils")
    utils.__path__ = []
    utils.is_multimodal = lambda: _multimodal[0]
    pkg.utils = utils
    sys.modules["mindspeed_rl"] = pkg
    sys.modules["mindspeed_rl.utils"] = utils
    spec = importlib.util.spec_from_file_location("mindspeed_rl.utils.seqlen_balancing", REFERENCE_FILE)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def plain(x):
    """Partitions as nested lists of python ints (the reference may hand back tensors or tuples)."""
    if isinstance(x, (list, tuple)):
        return [plain(v) for v in x]
    return int(x)


def lengths(rng, n, kind):
    if kind == "ties":            # few distinct values: almost every comparison is a tie
        return [rng.choice([3, 5, 5, 8, 8, 8, 13]) for _ in range(n)]
    if kind == "equal":
        return [rng.choice([7, 64])] * n
    if kind == "wide":            # response-like lengths
        return [rng.randint(1, 4096) for _ in range(n)]
    if kind == "steps":           # multiples of 128, as padded sequences are
        return [128 * rng.randint(1, 24) for _ in range(n)]
    raise ValueError(kind)


def main():
    ref = load_reference()
    rng = random.Random(20250131)
    cases = []
    for kind in ("ties", "equal", "wide", "steps"):
        for n in (1, 2, 3, 5, 8, 13, 16, 31) + ((64,) if kind == "ties" else ()):
            seq = lengths(rng, n, kind)
            for k in sorted({1, 2, 3, 4, 7, n}):
                if k > n:
                    continue
                for equal_size in (False, True):
                    if equal_size and n % k != 0:
                        continue
                    cases.append({"fn": "karmarkar_karp", "seqlen_list": seq, "k_partitions": k, "equal_size": equal_size,
                                  "out": plain(ref.karmarkar_karp(list(seq), k, equal_size))})
                    cases.append({"fn": "heapq_partition", "seqlen_list": seq, "k_partitions": k, "equal_size": equal_size,
                                  "out": plain(ref.heapq_partition(list(seq), k, equal_size))})
                    cases.append({"fn": "get_seqlen_balanced_partitions", "seqlen_list": seq, "k_partitions": k,
                                  "equal_size": equal_size,
                                  "out": plain(ref.get_seqlen_balanced_partitions(list(seq), k, equal_size))})
            longest, total = max(seq), sum(seq)
            for cap in sorted({longest, longest + 1, 2 * longest, max(longest, total // 3), total}):
                k0 = (total + cap - 1) // cap
                cases.append({"fn": "heapq_partition_with_max", "seqlen_list": seq, "k_partitions": k0, "max_token_len": cap,
                              "out": plain(ref.heapq_partition_with_max(list(seq), k0, cap))})
                for dyn in (None, 2, 5):
                    _multimodal[0] = False
                    cases.append({"fn": "rearrange_micro_batches", "seqlen_list": seq, "max_token_len": cap,
                                  "dynamic_max_batch_size": dyn, "multimodal": False,
                                  "out": plain(ref.rearrange_micro_batches(list(seq), cap, dyn))})
                _multimodal[0] = True
                cases.append({"fn": "rearrange_micro_batches", "seqlen_list": seq, "max_token_len": cap,
                              "dynamic_max_batch_size": None, "multimodal": True,
                              "out": plain(ref.rearrange_micro_batches(list(seq), cap))})
                _multimodal[0] = False
                cases.append({"fn": "balanced_bin_packing", "seqlen_list": seq, "max_capacity": cap,
                              "out": plain(ref.balanced_bin_packing(list(seq), cap))})
    for perm_n in (1, 2, 7, 32):
        perm = list(range(perm_n))
        rng.shuffle(perm)
        cases.append({"fn": "get_reverse_idx", "idx_map": perm, "out": plain(ref.get_reverse_idx(list(perm)))})
    doc = {"source": "outputs of /root/reference/mindspeed_rl/utils/seqlen_balancing.py executed by "
                     "tests/golden/make_reference_partition_vectors.py (data-parallel size 1, no process group)",
           "cases": cases}
    with open(OUT, "w") as fh:
        json.dump(doc, fh, separators=(",", ":"))
        fh.write("\n")
    print("wrote %d cases, %d bytes" % (len(cases), os.path.getsize(OUT)))


if __name__ == "__main__":
    main()
