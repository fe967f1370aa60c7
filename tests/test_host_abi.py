"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol the header
declares, its argument validation rejects bad calls without launching anything, and the Python
mirror keeps the reference's registry / meta-info / error contracts.  No kernel runs here."""
import ctypes
import os
import re

import pytest
import torch

import mindspeed_rl_amd as mrl
from mindspeed_rl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mrl_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mrl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 16
    for name in declared:
        assert hasattr(lib, name), "libmrl_hip.so lacks %s" % name
    # and the ctypes table binds exactly the declared set
    assert sorted(_lib.SIGNATURES) == declared
    assert lib.mrl_version() == 300
    # what the driver's build check compares against is read from the header, not a literal of its own
    import __graft_entry__
    assert __graft_entry__.header_version() == lib.mrl_version()
    assert lib.mrl_last_error() == b""
    assert os.path.dirname(_lib.library_path()).startswith(ROOT), "the library must live in-tree"


def test_header_is_plain_c_and_arities_match(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 without any other include path, and the
    ctypes table must pass as many arguments as each declaration takes."""
    import shutil
    import subprocess
    header = os.path.join(ROOT, "include", "mrl_hip.h")
    gcc = shutil.which("gcc")
    if gcc:
        src = tmp_path / "use_header.c"
        src.write_text('#include "mrl_hip.h"\nint (*probe)(void) = mrl_version;\nint main(void) { return probe == 0; }\n')
        subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-I",
                        os.path.dirname(header), str(src)], check=True)
    text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
    for name, params in re.findall(r"\b(mrl_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        n = 0 if params.strip() in ("", "void") else params.count(",") + 1
        assert len(_lib.SIGNATURES[name]) == n, name


def test_argument_validation_launches_nothing():
    lib = _lib.load()
    # NULL logits
    rc = lib.mrl_vocab_logprob_fwd(None, _lib.BF16, 4, 128, 128, None, _lib.I64, None, 1.0, None, None, None, None)
    assert rc == -1 and b"NULL" in lib.mrl_last_error()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 15) // 16 * 16
    # unsupported logits dtype
    rc = lib.mrl_vocab_logprob_fwd(p, _lib.I64, 4, 128, 128, p, _lib.I64, None, 1.0, p, None, None, None)
    assert rc == -2 and b"dtype" in lib.mrl_last_error()
    # stride below vocab
    rc = lib.mrl_vocab_logprob_fwd(p, _lib.BF16, 4, 128, 64, p, _lib.I64, None, 1.0, p, None, None, None)
    assert rc == -1 and b"row_stride" in lib.mrl_last_error()
    # misaligned fp32 logits
    rc = lib.mrl_vocab_logprob_fwd(p + 2, _lib.F32, 1, 8, 8, p, _lib.I64, None, 1.0, p, None, None, None)
    assert rc == -3
    # bad temperature
    rc = lib.mrl_vocab_logprob_fwd(p, _lib.BF16, 1, 8, 8, p, _lib.I64, None, 0.0, p, None, None, None)
    assert rc == -1 and b"inv_temperature" in lib.mrl_last_error()
    # negative rows
    rc = lib.mrl_vocab_logprob_fwd(p, _lib.BF16, -1, 8, 8, p, _lib.I64, None, 1.0, p, None, None, None)
    assert rc == -1
    # zero rows is a no-op success
    assert lib.mrl_vocab_logprob_fwd(None, _lib.BF16, 0, 8, 8, None, _lib.I64, None, 1.0, None, None, None, None) == 0
    # backward: g_entropy without the forward's entropy, mixed dtypes, partial overlap
    rc = lib.mrl_vocab_logprob_bwd(p, _lib.BF16, 2, 8, 8, p, _lib.I64, 1.0, p, None, p, p, p + 2048, _lib.BF16, 8, None)
    assert rc == -1 and b"g_entropy" in lib.mrl_last_error()
    rc = lib.mrl_vocab_logprob_bwd(p, _lib.F32, 2, 8, 8, p, _lib.I64, 1.0, p, None, p, None, p + 2048, _lib.BF16, 8, None)
    assert rc == -2
    rc = lib.mrl_vocab_logprob_bwd(p, _lib.BF16, 2, 8, 8, p, _lib.I64, 1.0, p, None, p, None, p + 16, _lib.BF16, 8, None)
    assert rc == -1 and b"overlap" in lib.mrl_last_error()
    # index maps
    assert lib.mrl_pack_index_build(None, _lib.I64, 4, 8, 0, p, p, None, None) == -1       # align 0
    assert lib.mrl_pack_index_build(None, _lib.I64, 4, 8, 1, p, None, None, None) == -1    # NULL cu
    assert lib.mrl_pack_rows(p, p, None, None, 3, 1, 8, p, p, 8, None, None) == -2         # elem_bytes 3
    assert lib.mrl_unpad_gather(p, 4, 8, 1, p, p, p, _lib.F32, 1, 8, p, None) == -2        # prompt dtype
    assert lib.mrl_group_advantage(p, _lib.F32, 6, 4, p, _lib.F32, 3, p, None, None) == -1  # 6 % 4
    assert b"multiple" in lib.mrl_last_error()
    assert lib.mrl_group_keep_mask(p, _lib.I32, 4, 2, p, None) == -2
    assert lib.mrl_policy_loss_fwd(p, None, None, p, None, None, 0, None, 0, 2, 4, 0.8, 1.2, 4, 0.0, 0.0, 0, 1.0, p, p,
                                   None) == -1                                             # no mask, no lengths
    assert lib.mrl_policy_loss_fwd(p, None, None, p, None, p, _lib.F32, None, 0, 2, 4, 0.8, 1.2, 4, 0.0, 0.0, 0, 1.0, p,
                                   p, None) == -1                                          # low_var_kl without ref
    assert b"ref_log_prob" in lib.mrl_last_error()
    assert lib.mrl_policy_loss_fwd(p, None, None, p, None, p, _lib.F32, None, 0, 2, 4, 0.8, 1.2, 9, 0.0, 0.0, 0, 1.0, p,
                                   p, None) == -1                                          # kl enum
    assert lib.mrl_copy_bytes(p, p + 1024, 24, None) == -1
    # fused sweep: a vocabulary the registers cannot hold, one that is not a whole number of vectors
    assert lib.mrl_fused_max_vocab(_lib.BF16) == 311296 and lib.mrl_fused_max_vocab(_lib.I64) == 0
    assert lib.mrl_fused_max_vocab(_lib.F32) == 155648
    assert lib.mrl_fused_workspace_bytes(_lib.BF16, 100, 152064) == 16
    assert lib.mrl_fused_workspace_bytes(_lib.F32, 100, 152064) == 16 + 100 * 32
    assert lib.mrl_fused_workspace_bytes(_lib.BF16, 100, 311304) == 0
    # a row that two workgroups hold needs the workspace
    rc = lib.mrl_fused_logprob_loss(p, _lib.F32, 2, 152064, 152064, p, _lib.I64, 1.0, p, 1, 0.8, 1.2, 4, 0.0, 0.0, 1.0,
                                    None, p + (1 << 30), 152064, None, None, p, None, 0, 0, None)
    assert rc == -1 and b"workspace" in lib.mrl_last_error()
    rc = lib.mrl_fused_logprob_loss(p, _lib.F32, 2, 152064, 152064, p, _lib.I64, 1.0, p, 1, 0.8, 1.2, 4, 0.0, 0.0, 1.0,
                                    None, p, 152064, None, None, p, p, 64, 0, None)
    assert rc == -1 and b"workspace" in lib.mrl_last_error()                              # too small for two rows
    for vocab in (311304, 1003):
        rc = lib.mrl_fused_logprob_loss(p, _lib.BF16, 2, vocab, vocab, p, _lib.I64, 1.0, p, 1, 0.8, 1.2, 4, 0.0, 0.0,
                                        1.0, None, p, vocab, None, None, p, None, 0, 0, None)
        assert rc == -2, vocab
    assert lib.mrl_fused_logprob_loss(p, _lib.BF16, 2, 64, 64, p, _lib.I64, 1.0, None, 1, 0.8, 1.2, 4, 0.0, 0.0, 1.0,
                                      None, p, 64, None, None, p, None, 0, 0, None) == -1  # no row operands
    assert lib.mrl_fused_logprob_loss(p, _lib.BF16, 2, 64, 64, p, _lib.I64, 1.0, p, 1, 0.8, 1.2, 4, 0.0, 0.0, 1.0,
                                      None, p, 64, None, None, p, p + 2, 16, 0, None) == -3  # misaligned workspace
    assert lib.mrl_scale_rows(p, _lib.I32, 2, 64, 64, p, p, None) == -2
    assert lib.mrl_scale_rows(p, _lib.BF16, 2, 64, 64, p, None, None) == -1                # no applied scale
    assert lib.mrl_grad_scale_note(p, None, None, None, None) == -1
    assert lib.mrl_scale_rows_note(p, _lib.BF16, 2, 64, 64, p, None, None, None, None) == -1
    assert lib.mrl_scale_rows_note(p, _lib.BF16, 2, 64, 64, p, p + 4, None, None, None) == -3   # scale + counter: 8 bytes
    # the prepare step clears the sweep's workspace in whole 8-byte words
    assert lib.mrl_fused_loss_prepare(0, 0, 4, 8, None, None, 0, None, 0, None, 0, None, None, None, None, 0, 0, None,
                                      None, None, p, p, 12, None, 1.0, None, None) == -1
    assert lib.mrl_fused_loss_prepare(0, 0, 4, 0, None, None, 0, None, 0, None, 0, None, None, None, None, 0, 0, None,
                                      None, None, None, p, 16, None, 1.0, None, None) == -1     # nothing to prepare for
    # the bound of the wide rows' wait: set, read back, restore
    assert lib.mrl_set_wide_spin_limit(0) == 1 << 18 and lib.mrl_set_wide_spin_limit(-1) == 0
    assert lib.mrl_set_wide_spin_limit(-1) == 1 << 18
    # fused lm_head: hidden size must be a multiple of the K tile, workspace must be large enough
    assert lib.mrl_lmhead_workspace_bytes(100, 1000) > 0
    assert lib.mrl_lmhead_logprob_fwd(p, p, 4, 1000, 100, p, _lib.I64, 1.0, p, None, None, p, 1 << 20, None) != 0
    assert lib.mrl_lmhead_logprob_fwd(p, p, 4, 1000, 128, p, _lib.I64, 1.0, p, None, None, p, 16, None) != 0
    assert b"workspace" in lib.mrl_last_error()
    # products of the lm_head training step
    assert lib.mrl_lmhead_logits(p, p, 4, 1000, 100, p, 1000, None) == -2                   # hidden_dim % 64
    assert lib.mrl_lmhead_logits(p, p, 4, 1001, 128, p, 1008, None) == -2                   # vocab % 8
    assert lib.mrl_lmhead_logits(p, p, 4, 1000, 128, p, 992, None) == -1                    # row stride below vocab
    assert lib.mrl_lmhead_logits(None, None, 0, 1000, 128, None, 1000, None) == 0
    assert lib.mrl_lmhead_logprob_bwd(p, p, p, 1000, 4, 1000, 128, p, p, None) == -1        # stride not a multiple of 64
    assert b"dlogits_row_stride" in lib.mrl_last_error()
    assert lib.mrl_lmhead_logprob_bwd(p, p, p, 1024, 4, 1000, 128, p, None, None) == -1     # NULL dWeight
    assert lib.mrl_lmhead_logprob_bwd(p, p, p, 1024, 4, 1004, 128, p, p, None) == -2        # vocab % 8
    assert lib.mrl_lmhead_logprob_bwd(None, None, None, 1024, 0, 1000, 128, None, None, None) == 0
    # PPO value side
    assert lib.mrl_gae_scan(p, p + 512, 2, 8, 1.0, 0.95, p, p + 1024, None) == -1 and b"alias" in lib.mrl_last_error()
    assert lib.mrl_gae_scan(p, p + 512, 2, 0, 1.0, 0.95, p + 1024, p + 2048, None) == -1
    assert lib.mrl_gae_scan(None, None, 0, 8, 1.0, 0.95, None, None, None) == 0
    assert lib.mrl_kl_token_rewards(p, p, p, _lib.I64, p, 2, 8, 0, 0.1, p, p, None) == -1   # no such penalty
    assert lib.mrl_kl_token_rewards(p, p, p, _lib.F32, p, 2, 8, 1, 0.1, p, p, None) == -2   # lengths dtype
    assert lib.mrl_masked_whiten(p, p, _lib.F64, 8, 1, p, p, None) == -2
    assert lib.mrl_masked_whiten(p, p, _lib.F32, 8, 1, p, None, None) == -1
    assert lib.mrl_value_loss_fwd(p, p, p, None, 0, None, 0, 2, 4, 0.5, 1.0, p, None) == -1  # no mask, no lengths
    assert lib.mrl_value_loss_bwd(p, p, p, p, _lib.F32, None, 0, 2, 4, 0.5, 1.0, p, None, p, None) == -1
    # bandwidth probe
    assert lib.mrl_bandwidth_probe(6, p, p, 1, 1024, None) == -1
    assert lib.mrl_bandwidth_probe(2, p, p, 1, 1000, None) == -1
    assert lib.mrl_bandwidth_probe(2, p, p, 1, 19 * 1024 * 16 + 16, None) == -2
    assert lib.mrl_bandwidth_probe(2, None, p, 1, 1024, None) == -1
    assert lib.mrl_bandwidth_probe(2, None, None, 0, 1024, None) == 0
    with pytest.raises(_lib.MrlError) as err:
        _lib.call("mrl_copy_bytes", p, p + 1024, 24, None)
    assert err.value.code == -1 and "multiple of 16" in str(err.value)


def test_cpu_tensors_are_refused_loudly():
    z = torch.randn(2, 8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mrl.compute_log_probs(z, torch.zeros(2, dtype=torch.long))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mrl.compute_group_norm_advantage_return(torch.ones(2, 1), torch.ones(2, 3), torch.ones(2, 1), 2)


def test_registry_contract(reference_vectors):
    assert isinstance(mrl.LossFuncFactory.get_instance("ray_grpo", "actor"), mrl.GRPOActorLossFunc)
    key = reference_vectors["dapo_defaults"]["registry_key"]
    assert isinstance(mrl.LossFuncFactory.get_instance(*key), mrl.DAPOActorLossFunc)
    assert isinstance(mrl.LossFuncFactory.get_instance("ray_ppo", "actor"), mrl.PPOActorLossFunc)
    assert isinstance(mrl.LossFuncFactory.get_instance("ray_ppo", "critic"), mrl.CriticLossFunc)
    assert isinstance(mrl.LossFuncFactory.get_instance("ray_grpo", "reference"), mrl.ReferenceLossFunc)
    assert isinstance(mrl.LossFuncFactory.get_instance("ray_ppo", "reference"), mrl.ReferenceLossFunc)
    assert mrl.LossFuncFactory.get_instance("nope", "actor") is None
    assert mrl.LossFuncFactory.get_class("ray_dapo", "actor") is mrl.DAPOActorLossFunc
    # the factory's map is its own: the base register stays empty
    assert "ray_grpo_actor" not in mrl.LossRegister.class_map

    @mrl.LossFuncFactory.register_loss("unit", "test")
    class Dummy(mrl.BaseLossFunc):
        def compute_loss(self, output, batch, forward_only=False, non_loss_data=True, **kwargs):
            return None

    assert isinstance(mrl.LossFuncFactory.get_instance("unit", "test"), Dummy)

    @mrl.LossFuncFactory.register_loss("unit", "test")
    class Dummy2(Dummy):
        pass

    assert isinstance(mrl.LossFuncFactory.get_instance("unit", "test"), Dummy2)   # re-registering overwrites
    del mrl.LossFuncFactory.class_map["unit_test"]
    with pytest.raises(TypeError):
        mrl.BaseLossFunc()        # abstract


def test_meta_info_contract(reference_vectors):
    d = reference_vectors["dapo_defaults"]
    f = mrl.DAPOActorLossFunc()
    assert f.clip_ratio == d["clip_ratio"] and f.entropy_coeff == d["entropy_coeff"]
    assert hasattr(f, "logprob_computer")
    for name in d["unset_until_meta"]:
        assert not hasattr(f, name)
    f.add_loss_meta_info(None)
    f.add_loss_meta_info({"clip_ratio": "0.3", "kl_ctrl": 0.1, "entropy_coeff": 0.01, "token_level_loss": 1,
                          "clip_higher_enable": 0, "clip_ratio_low": 0.1, "clip_ratio_high": 0.28, "beta": 3,
                          "unknown": 1})
    assert f.clip_ratio == 0.3 and f.kl_ctrl == 0.1 and f.entropy_coeff == 0.01
    assert f.token_level_loss is True and f.clip_higher_enable is False
    assert f.clip_ratio_low == 0.1 and f.clip_ratio_high == 0.28
    assert not hasattr(f, "beta") and not hasattr(f, "unknown")
    g = mrl.GRPOActorLossFunc()
    assert g.clip_ratio == 0.2 and g.entropy_coeff == 0.0 and not hasattr(g, "kl_ctrl")
    g.add_loss_meta_info({"clip_ratio": 0.25, "kl_ctrl": mrl.FixedKLController(0.001), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.0, "token_level_loss": True})
    assert g.clip_ratio == 0.25 and g.kl_ctrl.value == 0.001 and g.kl_penalty == "low_var_kl"
    assert not hasattr(g, "token_level_loss")
    assert mrl.FixedKLController(0.5).update(10, 20) is None
    # the vocab-op hook keeps its getter / setter
    assert mrl.get_vocab_parallel() is None
    mrl.set_vocab_parallel(mrl.vocab_parallel_cross_entropy)
    assert mrl.get_vocab_parallel() is mrl.vocab_parallel_cross_entropy
    mrl.set_vocab_parallel(None)
    mrl.set_parallel_state("x")
    assert mrl.get_parallel_state() == "x"
    mrl.set_parallel_state(None)


def test_host_side_error_contracts():
    with pytest.raises(ValueError, match="shape\\[0\\] == 1"):
        mrl.postprocess_packed_seqs(torch.zeros(2, 5), torch.zeros(2, dtype=torch.int32),
                                    torch.zeros(3, dtype=torch.int32), 4)
    with pytest.raises(ValueError, match="attention_mask_1d"):
        mrl.preprocess_packed_seqs(torch.zeros(2, 5, dtype=torch.long), torch.zeros(2, 5, dtype=torch.long),
                                   torch.zeros(2, 4, dtype=torch.long), 1)
    with pytest.raises(NotImplementedError):
        mrl.compute_kl_penalty(torch.zeros(1), torch.zeros(1), "full")
    with pytest.raises(NotImplementedError):
        mrl.policy_loss(torch.zeros(1, 1), None, None, None, torch.zeros(1, 1), mask=torch.ones(1, 1),
                        clip_low=0.2, clip_high=0.2, kl_penalty="full")
    with pytest.raises(NotImplementedError):
        mrl.vocab_parallel_cross_entropy(torch.zeros(1, 4), torch.zeros(1, dtype=torch.long), label_smoothing=0.1)
    # masked_mean stand-alone keeps the reference's vector
    assert mrl.masked_mean(torch.tensor([1.0, 2.0, 3.0]), torch.tensor([1.0, 0.0, 1.0]), epsilon=0) == 2.0
    assert mrl.compute_kl_penalty(torch.tensor([[0.5, 1.0]]), torch.tensor([[1.0, 0.5]])).tolist() == \
        [[0.14872121810913086, 0.10653066635131836]]


def test_multimodal_switch_selects_strategy_and_partitioner(monkeypatch):
    """The reference's process-wide switch (utils/utils.py:719-720, read in base_loss_func.py:15 and
    utils/seqlen_balancing.py:358): the environment variable IS_MULTIMODAL as a python literal."""
    from mindspeed_rl_amd import seqlen_balancing as sb
    monkeypatch.delenv("IS_MULTIMODAL", raising=False)
    assert mrl.is_multimodal() is False
    assert type(mrl.GRPOActorLossFunc().logprob_computer) is mrl.StandardLogProbComputer
    lengths = [90, 80, 70, 30, 20, 10]
    plain = sb.rearrange_micro_batches(lengths, 100)
    monkeypatch.setenv("IS_MULTIMODAL", "True")
    assert mrl.is_multimodal() is True
    for klass in (mrl.GRPOActorLossFunc, mrl.DAPOActorLossFunc, mrl.PPOActorLossFunc, mrl.ReferenceLossFunc):
        assert type(klass().logprob_computer) is mrl.MultimodalLogProbComputer
    packed = sb.rearrange_micro_batches(lengths, 100)
    assert packed == sb.balanced_bin_packing(lengths, 100)
    assert sb.rearrange_micro_batches(lengths, 100, multimodal=False) == plain
    monkeypatch.setenv("IS_MULTIMODAL", "False")
    assert type(mrl.GRPOActorLossFunc().logprob_computer) is mrl.StandardLogProbComputer


def test_deferred_stats_behaves_like_the_dict_of_floats_it_stands_for():
    """compute_loss(..., deferred_stats=True) returns a dict whose values are fetched from the device on
    first access: keys, len and `in` are known at once; every way to a value (indexing, items, values,
    get, dict(), {**x}, update, json, pickle, ==) synchronises once and then yields plain floats."""
    import json
    import pickle
    from mindspeed_rl_amd.loss import STAT_KEYS, DeferredStats

    class Event:
        waits = 0

        def synchronize(self):
            Event.waits += 1

    spec = [(STAT_KEYS[i], i + 1, i == 0) for i in range(5)]
    host = torch.tensor([9.0, -1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0])
    want = dict(zip(STAT_KEYS, [1.0, 2.0, 3.0, 4.0, 5.0]))           # abs() on the policy loss

    def fresh():
        return DeferredStats(spec, host, Event())

    d = fresh()
    assert isinstance(d, dict) and len(d) == 5 and STAT_KEYS[2] in d and list(d) == list(STAT_KEYS) and Event.waits == 0
    assert d[STAT_KEYS[0]] == 1.0 and Event.waits == 1 and d[STAT_KEYS[4]] == 5.0 and Event.waits == 1
    assert dict(fresh()) == want and {**fresh()} == want and fresh() == want and fresh().copy() == want
    assert json.loads(json.dumps(fresh())) == want
    restored = pickle.loads(pickle.dumps(fresh()))
    assert type(restored) is dict and restored == want
    merged = {}
    merged.update(fresh())
    assert merged == want and sorted(fresh().values()) == [1.0, 2.0, 3.0, 4.0, 5.0]
    assert fresh().get("absent", 7) == 7 and fresh().get(STAT_KEYS[1]) == 2.0
    assert all(isinstance(v, float) for _, v in fresh().items())
    assert "actor/pg_loss" in repr(fresh())
    # the form handed out under graph capture (no event): bound to the scalars themselves, read afresh on
    # every access, so that it shows what the latest replay left there
    live = DeferredStats(spec, host.clone(), None)
    assert dict(live) == want
    live._pending[1].mul_(2.0)
    assert live[STAT_KEYS[1]] == 4.0 and dict(live) == {k: 2.0 * v for k, v in want.items()}
