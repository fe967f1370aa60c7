"""Pins the CPU oracle before anything is compared with it: the reference's own unit-test
vectors, closed forms, invariants and brute force on tiny inputs.  Each check is chosen so
that a plausible slip (dropped term, wrong sign or index, biased instead of unbiased std,
transposed operand) fails it."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import advantage, loss, packing, vocab


# ----------------------------------------------------------------------------- reference-held vectors
def test_kl_penalty_reference_vectors(reference_vectors):
    v = reference_vectors["kl_penalty"]
    lp, ref = torch.tensor(v["logp"]), torch.tensor(v["ref_logp"])
    assert torch.allclose(loss.compute_kl_penalty(lp, ref, "kl"), torch.tensor(v["kl"]))
    assert torch.allclose(loss.compute_kl_penalty(lp, ref, "abs"), torch.tensor(v["abs"]))
    assert torch.allclose(loss.compute_kl_penalty(lp, ref, "mse"), torch.tensor(v["mse"]))
    assert loss.compute_kl_penalty(lp, ref, "low_var_kl").tolist() == v["low_var_kl_exact"]
    with pytest.raises(NotImplementedError):
        loss.compute_kl_penalty(lp, ref, "full")
    with pytest.raises(NotImplementedError):
        loss.compute_kl_penalty(lp, ref, "something-else")


def test_group_norm_reference_vector(reference_vectors):
    v = reference_vectors["group_norm_advantage"]
    adv, ret = advantage.compute_group_norm_advantage_return(
        torch.tensor(v["token_level_rewards"]), torch.tensor(v["eos_mask"]),
        torch.tensor(v["response_length"]), v["n_sample_per_prompt"])
    assert adv.shape == (2, 2) and adv.dtype == torch.float32
    assert torch.allclose(adv, torch.tensor(v["advantages"]), atol=1e-4)
    assert torch.allclose(ret, torch.tensor(v["returns"]), atol=1e-4)
    # the biased (population) std would give +-1.0: the vector tells the two apart
    assert abs(abs(adv[0, 0].item()) - 1.0) > 0.2
    # closed form for a two-sample group: +-(d/2) / (|d|/sqrt2 + 1e-6)
    expect = 0.5 / (1 / math.sqrt(2) + 1e-6)
    assert adv[1, 0].item() == pytest.approx(expect, abs=1e-7)


def test_masked_mean_reference_vector(reference_vectors):
    v = reference_vectors["masked_mean"]
    out = loss.masked_mean(torch.tensor(v["values"]), torch.tensor(v["mask"]), epsilon=v["epsilon"])
    assert out == v["expected"]
    # NaN outside the mask must not leak; default epsilon is 1e-8
    vals = torch.tensor([1.0, float("nan"), 3.0])
    assert loss.masked_mean(vals, torch.tensor(v["mask"])).item() == pytest.approx(2.0, abs=1e-6)
    # axis form
    m2 = torch.tensor([[1.0, 1.0], [0.0, 1.0]])
    v2 = torch.tensor([[1.0, 3.0], [5.0, 7.0]])
    assert torch.allclose(loss.masked_mean(v2, m2, axis=-1), torch.tensor([2.0, 7.0]))


def test_generate_mask_reference_vector(reference_vectors):
    v = reference_vectors["generate_mask"]
    out = packing.generate_mask(torch.tensor(v["data_pad"]), torch.tensor(v["seq_lengths"]))
    assert out.dtype == torch.int64
    assert out.tolist() == v["expected"]
    # lengths may arrive as [B,1]; zero length gives an all-zero row; over-long is all ones
    out = packing.generate_mask(torch.zeros(3, 4), torch.tensor([[0], [4], [9]]))
    assert out.tolist() == [[0, 0, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1]]


def test_truncate_middle_reference_vector(reference_vectors):
    v = reference_vectors["truncate_middle_and_pad"]
    out = packing.truncate_middle_and_pad(torch.tensor(v["responses"]), torch.tensor(v["input_tensor"]),
                                          torch.tensor(v["truncate_lengths"]), v["pad_value"])
    assert torch.allclose(out, torch.tensor(v["expected"]))


# ----------------------------------------------------------------------------- vocab ops
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_logprob_matches_textbook(dtype):
    g = torch.Generator().manual_seed(1)
    z = (torch.randn(1, 37, 501, generator=g) * 3).to(dtype)
    y = torch.randint(0, 501, (1, 37), generator=g)
    keep = z.clone()
    lp = vocab.compute_log_probs(z, y)
    assert torch.equal(z, keep), "compute_log_probs must not clobber its input"
    assert lp.dtype == torch.float32 and lp.shape == (1, 37)
    ref = torch.log_softmax(z.float(), -1).gather(-1, y.unsqueeze(-1)).squeeze(-1)
    assert torch.allclose(lp, ref, atol=2e-6)
    ce = torch.nn.functional.cross_entropy(z.float().view(-1, 501), y.view(-1), reduction="none")
    assert torch.allclose(lp.view(-1), -ce, atol=2e-6)
    lp64, _, _ = vocab.logprob_entropy_fp64(z, y)
    assert torch.allclose(lp.double(), lp64, atol=5e-6)


def test_logprob_invariants_and_special_cases():
    g = torch.Generator().manual_seed(2)
    z = torch.randn(5, 64, generator=g) * 4
    y = torch.randint(0, 64, (5,), generator=g)
    base = vocab.compute_log_probs(z, y)
    assert torch.allclose(vocab.compute_log_probs(z + 7.25, y), base, atol=1e-5)       # shift invariance
    uni = vocab.compute_log_probs(torch.zeros(3, 64), torch.tensor([0, 5, 63]))
    assert torch.allclose(uni, torch.full((3,), -math.log(64)), atol=1e-6)              # uniform
    # a wrong label index must be caught: permuting the label changes the answer
    assert not torch.allclose(vocab.compute_log_probs(z, (y + 1) % 64), base)
    # sum_j exp(logp_j) == 1 over all labels of one row
    allp = vocab.compute_log_probs(z[:1].expand(64, 64).contiguous(), torch.arange(64))
    assert allp.exp().sum().item() == pytest.approx(1.0, abs=1e-5)
    # a label outside [0, V) is masked like Megatron does: predicted logit 0 after the max shift
    bad = vocab.compute_log_probs(z[:2], torch.tensor([-1, 64]))
    zz = z[:2] - z[:2].max(-1, keepdim=True).values
    assert torch.allclose(bad, -zz.exp().sum(-1).log(), atol=1e-6)


def test_entropy_matches_categorical():
    g = torch.Generator().manual_seed(3)
    z = torch.randn(1, 21, 333, generator=g) * 2
    h = vocab.vocab_parallel_entropy(z.clone())
    ref = torch.distributions.Categorical(logits=z).entropy()
    assert torch.allclose(h, ref, atol=1e-5)
    _, h64, _ = vocab.logprob_entropy_fp64(z, torch.zeros(1, 21, dtype=torch.long))
    assert torch.allclose(h.double(), h64, atol=1e-5)
    assert (h >= 0).all() and (h <= math.log(333) + 1e-6).all()
    assert vocab.vocab_parallel_entropy(torch.zeros(2, 128))[0].item() == pytest.approx(math.log(128), abs=1e-6)
    assert torch.allclose(vocab.vocab_parallel_entropy(z + 3.0), h, atol=1e-5)


def test_vocab_gradients():
    g = torch.Generator().manual_seed(4)
    z = (torch.randn(6, 40, generator=g) * 2).requires_grad_()
    y = torch.randint(0, 40, (6,), generator=g)
    w_lp = torch.randn(6, generator=g)
    w_h = torch.randn(6, generator=g)
    out = (vocab.compute_log_probs(z, y) * w_lp).sum() + (vocab.vocab_parallel_entropy(z) * w_h).sum()
    (gz,) = torch.autograd.grad(out, z)
    z2 = z.detach().clone().requires_grad_()
    lsm = torch.log_softmax(z2, -1)
    ref = (lsm.gather(-1, y[:, None]).squeeze(-1) * w_lp).sum() + \
        (torch.distributions.Categorical(logits=z2).entropy() * w_h).sum()
    (gref,) = torch.autograd.grad(ref, z2)
    assert torch.allclose(gz, gref, atol=1e-5)
    assert torch.allclose(gz.sum(-1), torch.zeros(6), atol=1e-5)       # both gradients sum to 0 per row
    # closed form: dz = g_lp (onehot - p) - g_H p (z - E_p z)
    p = torch.softmax(z.detach(), -1)
    onehot = torch.nn.functional.one_hot(y, 40).float()
    ez = (p * z.detach()).sum(-1, keepdim=True)
    closed = w_lp[:, None] * (onehot - p) - w_h[:, None] * p * (z.detach() - ez)
    assert torch.allclose(gz, closed, atol=1e-5)
    # fp64 gradcheck of both autograd functions
    zd = (torch.randn(3, 7, generator=g, dtype=torch.float64)).requires_grad_()
    yd = torch.tensor([0, 3, 6])
    assert torch.autograd.gradcheck(lambda t: vocab.vocab_parallel_entropy(t), (zd,), atol=1e-6)

    def lp64(t):
        # the CE restatement up-casts to fp32 by design; check it against fp64 finite differences loosely
        return vocab.compute_log_probs(t.float(), yd).double()
    num = torch.zeros(3, 7, dtype=torch.float64)
    eps = 1e-3
    for i in range(3):
        for j in range(7):
            d = torch.zeros(3, 7, dtype=torch.float64)
            d[i, j] = eps
            num[i, j] = (lp64(zd.detach() + d).sum() - lp64(zd.detach() - d).sum()) / (2 * eps)
    zf = zd.detach().float().requires_grad_()
    (an,) = torch.autograd.grad(vocab.compute_log_probs(zf, yd).sum(), zf)
    assert torch.allclose(an.double(), num, atol=2e-3)


# ----------------------------------------------------------------------------- packing
def _random_batch(g, batch, width, align):
    plen = torch.randint(1, 6, (batch, 1), generator=g, dtype=torch.int32)
    rlen = torch.randint(0, width - 6, (batch, 1), generator=g, dtype=torch.int32)
    ids = torch.randint(1, 1000, (batch, width), generator=g)
    total = plen + rlen
    mask = packing.generate_mask(ids, total)
    ids = ids * mask
    return ids, plen, rlen, mask


@pytest.mark.parametrize("align", [1, 2, 8])
def test_pack_unpack_brute_force(align):
    g = torch.Generator().manual_seed(10 + align)
    ids, plen, rlen, mask = _random_batch(g, 9, 40, align)
    labels = torch.cat([ids[:, 1:], torch.zeros(9, 1, dtype=ids.dtype)], dim=1)
    p_ids, p_pos, p_lab, seqlens, cu = packing.preprocess_packed_seqs(ids, labels, mask, align)
    assert seqlens.dtype == torch.int32 and cu.dtype == torch.int32
    assert seqlens.tolist() == (plen + rlen).flatten().tolist()
    # independent numpy restatement of the layout
    lens = (plen + rlen).flatten().numpy()
    padded = (lens + align - 1) // align * align
    cu_np = np.concatenate([[0], np.cumsum(padded)])
    assert cu.tolist() == cu_np.tolist()
    assert p_ids.shape == (1, int(cu_np[-1]))
    flat = np.zeros(int(cu_np[-1]), dtype=np.int64)
    pos = np.zeros(int(cu_np[-1]), dtype=np.int64)
    for i in range(9):
        flat[cu_np[i]:cu_np[i] + lens[i]] = ids[i, :lens[i]].numpy()
        pos[cu_np[i]:cu_np[i + 1]] = np.arange(padded[i])
    assert p_ids[0].tolist() == flat.tolist()
    assert p_pos[0].tolist() == pos.tolist()
    # unpack without prompt truncation restores every valid position
    back = packing.postprocess_packed_seqs(p_ids, seqlens, cu, 40)
    assert torch.equal(back, ids)
    # unpack with the prompt shift: row i holds packed[cu_i + P_i - 1 : cu_i + P_i - 1 + R_i]
    vals = torch.arange(p_ids.shape[1], dtype=torch.float32).unsqueeze(0)
    resp = packing.postprocess_packed_seqs(vals, seqlens, cu, 34, prompt_length=plen)
    for i in range(9):
        P, R = plen[i].item(), rlen[i].item()
        want = [float(cu_np[i] + P - 1 + k) for k in range(R)] + [0.0] * (34 - R)
        assert resp[i].tolist() == want
    with pytest.raises(ValueError):
        packing.postprocess_packed_seqs(torch.zeros(2, 5), seqlens, cu, 40)
    with pytest.raises(ValueError):
        packing.preprocess_packed_seqs(ids, labels, mask[:, :-1], align)


def test_padded_window_equals_packed_unpack():
    g = torch.Generator().manual_seed(20)
    ids, plen, rlen, mask = _random_batch(g, 7, 30, 1)
    vals = torch.randn(7, 30, generator=g)
    window = packing.response_window(plen, rlen)
    assert window.tolist() == [[p - 1, p + r - 1] for p, r in zip(plen.flatten().tolist(), rlen.flatten().tolist())]
    resp = torch.zeros(7, 24)
    out = packing.truncate_prompt_and_pad(resp, vals, window)
    _, _, _, seqlens, cu = packing.preprocess_packed_seqs(ids, ids, mask, 1)
    packed = torch.cat([vals[i, :seqlens[i]] for i in range(7)]).unsqueeze(0)
    out2 = packing.postprocess_packed_seqs(packed, seqlens, cu, 24, prompt_length=plen)
    assert torch.equal(out, out2)


# ----------------------------------------------------------------------------- policy loss
def _loss_inputs(g, rows=5, cols=9):
    lp = -torch.rand(rows, cols, generator=g) * 3
    old = lp + torch.randn(rows, cols, generator=g) * 0.3
    ref = lp + torch.randn(rows, cols, generator=g) * 0.3
    adv = torch.randn(rows, 1, generator=g).repeat(1, cols)
    ent = torch.rand(rows, cols, generator=g)
    lens = torch.randint(1, cols + 1, (rows,), generator=g)
    mask = packing.generate_mask(lp, lens)
    return lp, old, ref, adv, ent, mask


def test_grpo_loss_hand_cases():
    one = torch.ones(1, 4)
    mask = torch.tensor([[1, 1, 1, 0]])
    lp = torch.tensor([[-1.0, -2.0, -0.5, -9.0]])
    adv = torch.tensor([[0.5, -1.0, 2.0, 7.0]])
    # old=None: ratio 1, nothing clipped, pg = -mean(A) over the mask; ref == lp: kl 0
    out = loss.grpo_policy_loss(None, lp, lp.clone(), adv, torch.zeros_like(lp), mask, 0.2, 0.5, "low_var_kl", 0.0)
    assert out[0].item() == pytest.approx(-(0.5 - 1.0 + 2.0) / 3, abs=1e-6)
    assert out[1].item() == 0.0 and out[2].item() == 0.0 and out[3].item() == 0.0
    # forced clipping on each side of each sign of A (eps 0.2): ratio 2 and 0.5
    for ratio, a, expect_pg, clipped in [(2.0, 1.0, -1.2, True), (2.0, -1.0, 2.0, False),
                                         (0.5, 1.0, -0.5, False), (0.5, -1.0, 0.8, True)]:
        lpx = torch.full((1, 4), math.log(ratio))
        o = loss.grpo_policy_loss(torch.zeros(1, 4), lpx, lpx, a * one, torch.zeros(1, 4), one, 0.2, 0.0,
                                  "low_var_kl", 0.0)
        assert o[0].item() == pytest.approx(expect_pg, abs=1e-6)
        assert o[1].item() == pytest.approx(1.0 if clipped else 0.0, abs=1e-6)
        assert o[2].item() == pytest.approx(-math.log(ratio), abs=1e-6)
    # kl and entropy terms enter with +coef and -coef
    ref = lp - 0.5
    o = loss.grpo_policy_loss(None, lp, ref, torch.zeros_like(lp), torch.full_like(lp, 2.0), mask, 0.2, 0.1,
                              "low_var_kl", 0.01)
    k3 = math.exp(-0.5) + 0.5 - 1
    assert o[3].item() == pytest.approx(k3, abs=1e-6)
    assert o[0].item() == pytest.approx(0.1 * k3 - 0.01 * 2.0, abs=1e-6)
    assert o[4].item() == pytest.approx(2.0, abs=1e-6)


def test_policy_loss_gradient_rule():
    """dL/dlp of the clipped surrogate: -A*r/N unless (A>0 and r>1+eps) or (A<0 and r<1-eps)."""
    g = torch.Generator().manual_seed(30)
    lp, old, ref, adv, ent, mask = _loss_inputs(g, 6, 11)
    lp = lp.requires_grad_()
    out = loss.grpo_policy_loss(old, lp, ref, adv, ent, mask, 0.2, 0.0, "low_var_kl", 0.0)
    (glp,) = torch.autograd.grad(out[0], lp)
    r = torch.exp(lp.detach() - old)
    dead = ((adv > 0) & (r > 1.2)) | ((adv < 0) & (r < 0.8))
    n = mask.sum() + 1e-8
    want = torch.where(dead, torch.zeros_like(r), -adv * r) * mask / n
    assert torch.allclose(glp, want, atol=1e-7)
    # k3 gradient: -(exp(ref-lp) - 1) inside the clamps
    lp2 = lp.detach().clone().requires_grad_()
    out = loss.grpo_policy_loss(old, lp2, ref, torch.zeros_like(adv), ent, mask, 0.2, 1.0, "low_var_kl", 0.0)
    (gk,) = torch.autograd.grad(out[0], lp2)
    want = -(torch.exp(ref - lp2.detach()) - 1) * mask / n
    assert torch.allclose(gk, want, atol=1e-6)


def test_dapo_fixture_inputs(reference_vectors):
    v = reference_vectors["dapo_policy_loss_inputs"]
    t = {k: torch.tensor(v[k], dtype=torch.float32) for k in ("old_log_prob", "log_prob", "entropy", "advantages", "eos_mask")}
    r = math.exp(0.05)           # every ratio is exp(0.05), inside [0.9, 1.3]
    for token_level in (True, False):
        o = loss.dapo_policy_loss(t["old_log_prob"], t["log_prob"], t["entropy"], v["entropy_coeff"], t["advantages"],
                                  t["eos_mask"], v["clip_ratio_low"], v["clip_ratio_high"], token_level)
        ent = (0.01 + 0.02 + 0.04 + 0.05) / 4
        if token_level:
            pg = -(0.1 + 0.2 + 0.4 + 0.5) * r / 4
        else:
            pg = -((0.1 + 0.2) / 2 + (0.4 + 0.5) / 2) * r / 2
        assert o[0].item() == pytest.approx(pg - 0.01 * ent, abs=1e-6)
        assert o[1].item() == 0.0
        assert o[2].item() == pytest.approx(-0.05, abs=1e-6)
        assert o[3].item() == 0.0
        assert o[4].item() == pytest.approx(ent, abs=1e-7)
    o = loss.dapo_policy_loss(None, t["log_prob"], t["entropy"], v["entropy_coeff"], t["advantages"], t["eos_mask"],
                              v["clip_ratio_low"], v["clip_ratio_high"], False)
    assert o[0].item() == pytest.approx(-((0.1 + 0.2) / 2 + (0.4 + 0.5) / 2) / 2 - 0.01 * 0.03, abs=1e-6)
    # asymmetric clip: ratio 1.25 is clipped at eps_high 0.2 but not at 0.3
    lpx = torch.full((1, 2), math.log(1.25))
    ones = torch.ones(1, 2)
    o = loss.dapo_policy_loss(torch.zeros(1, 2), lpx, ones * 0, 0.0, ones, ones, 0.2, 0.2, True)
    assert o[1].item() == 1.0 and o[0].item() == pytest.approx(-1.2, abs=1e-6)
    o = loss.dapo_policy_loss(torch.zeros(1, 2), lpx, ones * 0, 0.0, ones, ones, 0.2, 0.3, True)
    assert o[1].item() == 0.0 and o[0].item() == pytest.approx(-1.25, abs=1e-6)
    # sequence-mean with an all-masked row is NaN in the reference (0/0); kept
    o = loss.dapo_policy_loss(torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2), 0.0, torch.ones(2, 2),
                              torch.tensor([[1.0, 1.0], [0.0, 0.0]]), 0.2, 0.2, False)
    assert math.isnan(o[0].item())


# ----------------------------------------------------------------------------- advantages / filter
def test_group_norm_closed_forms():
    g = torch.Generator().manual_seed(40)
    rewards = torch.randn(12, 1, generator=g)
    mask = packing.generate_mask(torch.zeros(12, 5), torch.randint(0, 6, (12,), generator=g))
    adv, ret = advantage.compute_group_norm_advantage_return(rewards, mask, torch.zeros(12, 1), 4)
    r = rewards.double().reshape(3, 4)
    want = ((r - r.mean(1, keepdim=True)) / (torch.std(r, dim=1, keepdim=True, unbiased=True) + 1e-6)).reshape(12, 1).float()
    assert torch.equal(adv, want.repeat(1, 5) * mask)
    assert torch.equal(ret, adv) and ret is not adv
    # all-equal rewards give exactly zero (std 0 handled by the eps)
    adv, _ = advantage.compute_group_norm_advantage_return(torch.ones(4, 1), torch.ones(4, 3), torch.zeros(4, 1), 4)
    assert torch.equal(adv, torch.zeros(4, 3))
    # group id is row // G: swapping two rows of different groups changes both groups
    r2 = rewards.clone()
    r2[[0, 4]] = r2[[4, 0]]
    adv2, _ = advantage.compute_group_norm_advantage_return(r2, torch.ones(12, 1), torch.zeros(12, 1), 4)
    adv1, _ = advantage.compute_group_norm_advantage_return(rewards, torch.ones(12, 1), torch.zeros(12, 1), 4)
    assert not torch.allclose(adv1[:8], adv2[:8]) and torch.equal(adv1[8:], adv2[8:])


def test_dynamic_sampling_predicate():
    vals = [1, 1, 1, 1, 0, 1, 0, 0, 0.5, 0.5, 0.5, 0.5, 0, 0, 0, 1e-100]
    assert advantage.dynamic_sampling_keep(vals, 4) == [4, 5, 6, 7, 12, 13, 14, 15]
    # numpy's arithmetic decides, not "all equal": squares that underflow give std 0 (dropped),
    # and three equal 0.1 have a mean that rounds away from 0.1, so std > 0 (kept)
    assert advantage.dynamic_sampling_keep([0, 0, 0, 1e-300], 4) == []
    assert advantage.dynamic_sampling_keep([0.1, 0.1, 0.1], 3) == [0, 1, 2]
    assert advantage.dynamic_sampling_keep([0.1, 0.1, 0.1, 0.1], 4) == []
    assert advantage.dynamic_sampling_keep([3.0, 3.0], 1) == [0, 1]      # single-member groups are kept
    assert advantage.dynamic_sampling_keep([2.0, 2.0], 2) == []


def test_compute_loss_end_to_end_shapes():
    g = torch.Generator().manual_seed(50)
    B, S, V, L = 4, 12, 50, 8
    plen = torch.tensor([[2], [3], [1], [4]], dtype=torch.int32)
    rlen = torch.tensor([[5], [8], [0], [3]], dtype=torch.int32)
    ids = torch.randint(0, V, (B, S), generator=g)
    mask1d = packing.generate_mask(ids, plen + rlen)
    labels = torch.cat([ids[:, 1:], torch.zeros(B, 1, dtype=ids.dtype)], 1)
    p_ids, _, p_lab, seqlens, cu = packing.preprocess_packed_seqs(ids, labels, mask1d, 2)
    T = p_ids.shape[1]
    logits = torch.randn(1, T, V, generator=g, requires_grad=True)
    batch = {"labels": p_lab, "responses": torch.zeros(B, L, dtype=torch.int32), "response_length": rlen,
             "prompt_length": plen, "advantages": torch.randn(B, 1, generator=g).repeat(1, L),
             "old_log_prob": -torch.rand(B, L, generator=g), "ref_log_prob": -torch.rand(B, L, generator=g)}
    kw = dict(use_remove_padding=True, seqlens_in_batch=seqlens, cu_seqlens_padded=cu)
    meta = dict(clip_ratio=0.2, kl_coef=0.001, kl_penalty="low_var_kl", entropy_coeff=0.001)
    lp = loss.grpo_compute_loss(logits, batch, meta, forward_only=True, **kw)
    assert lp.shape == (B, L)
    # packed and padded layouts agree
    padded_logits = torch.zeros(B, S, V)
    for i in range(B):
        padded_logits[i, :seqlens[i]] = logits[0, cu[i]:cu[i] + seqlens[i]].detach()
    batch_p = dict(batch, labels=labels)
    lp_p = loss.grpo_compute_loss(padded_logits, batch_p, meta, forward_only=True)
    assert torch.allclose(lp, lp_p, atol=1e-6)
    out, stats = loss.grpo_compute_loss(logits, batch, meta, **kw)
    assert out.dim() == 0 and set(stats) == {"actor/pg_loss", "actor/pg_clipfrac", "actor/ppo_kl", "actor/kl_loss", "actor/entropy"}
    assert stats["actor/pg_loss"] >= 0
    (gz,) = torch.autograd.grad(out, logits)
    assert gz.shape == logits.shape
    # rows that are not response rows get exactly zero gradient
    live = torch.zeros(T, dtype=torch.bool)
    for i in range(B):
        P, R = plen[i].item(), rlen[i].item()
        live[cu[i] + P - 1: cu[i] + P - 1 + R] = True
    assert torch.equal(gz[0, ~live], torch.zeros_like(gz[0, ~live]))
    assert (gz[0, live].abs().sum(-1) > 0).all()
    out2, _ = loss.grpo_compute_loss(logits, batch, meta, use_dynamic_bsz=True, actual_micro_batch_size=2.0, **kw)
    assert out2.item() == pytest.approx(out.item() * 2.0, rel=1e-6)
    d_out, d_stats = loss.dapo_compute_loss(logits, batch, dict(entropy_coeff=0.0, token_level_loss=True,
                                            clip_higher_enable=True, clip_ratio_low=0.2, clip_ratio_high=0.28), **kw)
    assert d_stats["actor/kl_loss"] == 0.0 and d_stats["actor/entropy"] == 0.0
    assert oracle.__doc__ and "TEST INFRASTRUCTURE" in oracle.__doc__


def test_wire_format_reference_vectors():
    """truncate_rows vector of the reference (tests/ut/utils/test_pad_process.py:64-72) and the worked example
    in the docstring of unpack_pad_experience (trainer/utils/transfer_dock.py:1096-1121)."""
    tensor = torch.tensor([[1, 2, 3, 4], [5, 6, 7, 8], [9, 10, 11, 12]])
    got = packing.truncate_rows(tensor, torch.tensor([[2], [3], [1]]))
    assert [r.tolist() for r in got] == [[1, 2], [5, 6, 7], [9]]
    assert [r.tolist() for r in packing.truncate_rows(tensor, torch.tensor([[2], [0], [1]]), left_pad=True)] == \
        [[3, 4], [5, 6, 7, 8], [12]]
    marked = torch.tensor([[-1, 0, 0], [4, 5, 6]])
    got = packing.truncate_rows(marked, torch.tensor([[0], [2]]))
    assert got[0].dtype == torch.int32 and got[0].numel() == 0 and got[1].tolist() == [4, 5]
    data = {"prompts": torch.tensor([1, 1, 1, 2, 2, 2, 2, 3, 3, 3, 4, 4, 4, 4]),
            "attention_mask": torch.tensor([1, 2, 2, 3, 3, 3, 4, 4, 4, 4])}
    lens = {"prompts": torch.tensor([3, 4, 3, 4], dtype=torch.int32),
            "attention_mask": torch.tensor([1, 2, 3, 4], dtype=torch.int32)}
    out = packing.unpack_pad_experience(data, lens, -1, 8)
    assert out["prompts"].tolist() == [[1, 1, 1, -1, -1, -1, -1, -1], [2, 2, 2, 2, -1, -1, -1, -1],
                                       [3, 3, 3, -1, -1, -1, -1, -1], [4, 4, 4, 4, -1, -1, -1, -1]]
    assert out["attention_mask"].tolist() == [[1, -1, -1, -1, -1, -1, -1, -1], [2, 2, -1, -1, -1, -1, -1, -1],
                                              [3, 3, 3, -1, -1, -1, -1, -1], [4, 4, 4, 4, -1, -1, -1, -1]]
    with pytest.raises(ValueError):
        packing.unpack_pad_experience({}, {}, 0, 1)
    with pytest.raises(ValueError):
        packing.unpack_pad_experience(data, {"prompts": lens["prompts"]}, 0, 1)
    # the worked example in the docstring of pack_experience_columns (transfer_dock.py:1015-1037): the
    # same columns as lists of samples pack to exactly the flat tensors and lengths above
    samples = {"prompts": [torch.tensor([1, 1, 1]), torch.tensor([2, 2, 2, 2]), torch.tensor([3, 3, 3]),
                           torch.tensor([4, 4, 4, 4])],
               "attention_mask": [torch.tensor([1]), torch.tensor([2, 2]), torch.tensor([3, 3, 3]),
                                  torch.tensor([4, 4, 4, 4])]}
    flat, flat_len = packing.pack_experience_columns("actor_train", samples, 4)
    for k in data:
        assert torch.equal(flat[k], data[k]) and torch.equal(flat_len[k], lens[k]) and flat_len[k].dtype == torch.int32
    pos = {"position_ids": [torch.arange(6).view(3, 2), torch.arange(9).view(3, 3) + 10]}
    flat, flat_len = packing.pack_experience_columns("actor_train", pos, 2)
    assert flat["position_ids"].tolist() == [[0, 1, 10, 11, 12], [2, 3, 13, 14, 15], [4, 5, 16, 17, 18]]
    assert flat_len["position_ids"].tolist() == [2, 3]
    back = packing.unpack_pad_experience(flat, flat_len, 0, 1)["position_ids"]
    assert back.shape == (2, 3, 3) and back[0, :, :2].tolist() == pos["position_ids"][0].tolist()
    with pytest.raises(ValueError):
        packing.pack_experience_columns("actor_train", samples, 3)
    with pytest.raises(ValueError):
        packing.pack_experience_columns("actor_train", {}, 0)


# --------------------------------------------------------------------------------- PPO value side
def test_value_side_reference_vectors(reference_vectors):
    """masked_var / masked_whiten (tests/ut/utils/test_torch_functional.py:36-55), GAE and the adaptive
    KL controller (tests/ut/utils/test_compute_utils.py:7-58), critic defaults and the no-clipping case
    (tests/ut/models/loss/test_critic_loss_func.py:28-141)."""
    v = reference_vectors["masked_var"]
    got = loss.masked_var(torch.tensor(v["values"]), torch.tensor(v["mask"]), unbiased=True)
    assert torch.isclose(got, torch.tensor(v["expected"]), atol=v["atol"])
    w = reference_vectors["masked_whiten"]
    got = loss.masked_whiten(torch.tensor(w["values"]), torch.tensor(w["mask"]))
    assert torch.allclose(got, torch.tensor(w["expected"]), atol=w["atol"])
    g = reference_vectors["gae"]
    adv, ret = advantage.compute_gae_advantage_return(torch.tensor(g["token_level_rewards"]), torch.tensor(g["values"]),
                                                      torch.tensor(g["eos_mask"]), torch.tensor(g["gamma"]),
                                                      torch.tensor(g["lam"]))
    assert torch.equal(adv, torch.tensor(g["expected_advantages"]))
    assert torch.equal(ret, torch.tensor(g["expected_returns"]))
    a = reference_vectors["adaptive_kl"]
    for case in a["cases"]:
        ctrl = advantage.AdaptiveKLController(a["init_kl_coef"], a["target_kl"], a["horizon"])
        ctrl.update(case["current_kl"], case["n_steps"])
        assert ctrl.value == case["expected"]
    c = reference_vectors["critic"]["no_clipping"]
    vf, frac = loss.value_loss(torch.tensor(c["vpreds"]), torch.tensor(c["returns"]), torch.tensor(c["values"]),
                               torch.tensor(c["response_mask"], dtype=torch.float32), c["cliprange_value"])
    assert frac.item() == c["expected_clipfrac"] and vf.item() == 0.0
    c = reference_vectors["critic"]["generic"]
    vf, frac = loss.value_loss(torch.tensor(c["vpreds"]), torch.tensor(c["returns"]), torch.tensor(c["values"]),
                               torch.tensor(c["response_mask"], dtype=torch.float32), c["cliprange_value"])
    # every masked error is 0.1: 0.5 * mean(0.01); vpreds == values, so nothing is clipped
    assert vf.item() == pytest.approx(0.005, rel=1e-5) and frac.item() == 0.0


def test_value_side_closed_forms():
    """What the mathematics fixes: GAE as the discounted sum of TD errors (fp64 brute force), lam = 1
    gives discounted returns, whitening gives zero masked mean and unit unbiased masked variance, the
    value loss in its three regimes (inside the clip range, clipped and worse, clipped and better) with
    the gradient of each, and the KL reward layout."""
    gen = torch.Generator().manual_seed(3)
    B, L = 5, 17
    r = torch.randn(B, L, generator=gen)
    v = torch.randn(B, L, generator=gen)
    mask = packing.generate_mask(r, torch.tensor([[17], [1], [9], [16], [2]])).float()
    gamma, lam = torch.tensor(0.97), torch.tensor(0.9)
    adv, ret = advantage.compute_gae_advantage_return(r, v, mask, gamma, lam)
    r64, v64 = r.double(), v.double()
    vn = torch.cat([v64[:, 1:], torch.zeros(B, 1, dtype=torch.float64)], 1)
    delta = r64 + 0.97 * vn - v64
    raw = torch.zeros(B, L, dtype=torch.float64)
    for t in range(L):
        for k in range(t, L):
            raw[:, t] += (float(gamma) * float(lam)) ** (k - t) * delta[:, k]
    assert (ret.double() - (raw + v64)).abs().max().item() < 1e-5
    want = loss.masked_whiten(raw.float(), mask)
    assert (adv - want).abs().max().item() < 1e-5
    n = mask.sum()
    assert abs((adv * mask).sum().item() / n.item()) < 1e-6
    assert ((adv * mask) ** 2).sum().item() / (n.item() - 1) == pytest.approx(1.0, rel=1e-4)
    # lam = 1: returns are the discounted reward-to-go (values cancel)
    _, ret1 = advantage.compute_gae_advantage_return(r, v, mask, torch.tensor(0.5), torch.tensor(1.0))
    togo = torch.zeros(B, L, dtype=torch.float64)
    for t in range(L):
        for k in range(t, L):
            togo[:, t] += 0.5 ** (k - t) * r64[:, k]
    assert (ret1.double() - togo).abs().max().item() < 1e-5
    # masked_var: biased / unbiased, one-element mask, empty mask raises
    x = torch.tensor([1.0, 5.0, 100.0])
    m = torch.tensor([1.0, 1.0, 0.0])
    assert loss.masked_var(x, m, unbiased=False).item() == pytest.approx(4.0)
    assert loss.masked_var(x, m).item() == pytest.approx(8.0)
    assert loss.masked_var(x, torch.tensor([0.0, 1.0, 0.0])).item() == pytest.approx(0.0)
    with pytest.raises(ValueError):
        loss.masked_var(x, torch.zeros(3))
    # value loss regimes, clip 0.5, value 0: vp 0.2 / ret 1 (inside), vp 2 / ret 3 (clipped to 0.5, worse:
    # takes the clipped error, no gradient), vp 2 / ret 0 (clipped, better: takes the raw error)
    vp = torch.tensor([[0.2, 2.0, 2.0, 9.0]], requires_grad=True)
    rt = torch.tensor([[1.0, 3.0, 0.0, 0.0]])
    vf, frac = loss.value_loss(vp, rt, torch.zeros(1, 4), torch.tensor([[1.0, 1.0, 1.0, 0.0]]), 0.5)
    assert vf.item() == pytest.approx(0.5 * (0.64 + 6.25 + 4.0) / 3, rel=1e-6)
    assert frac.item() == pytest.approx(1 / 3, rel=1e-6)
    (g,) = torch.autograd.grad(vf, vp)
    assert torch.allclose(g, torch.tensor([[0.5 * 2 * (0.2 - 1.0) / 3, 0.0, 0.5 * 2 * 2.0 / 3, 0.0]]), atol=1e-6)
    # KL rewards: score at the last response token, -beta * kl elsewhere, nothing past the response
    old = torch.tensor([[-1.0, -2.0, -3.0], [-1.0, -1.0, -1.0]])
    ref = torch.tensor([[-1.5, -2.0, -2.0], [-2.0, -2.0, -2.0]])
    rew, cur = advantage.kl_token_level_rewards(old, ref, torch.tensor([[2], [3]]), torch.tensor([10.0, -4.0]), 0.1, "kl")
    assert torch.allclose(rew, torch.tensor([[-0.05, 10.0, 0.0], [-0.1, -0.1, -4.1]]), atol=1e-6)
    assert cur == pytest.approx(0.5 * (0.25 + 1.0), rel=1e-6)
    out = loss.critic_compute_loss(torch.arange(12.0).view(2, 6, 1), {
        "responses": torch.zeros(2, 3), "prompt_length": torch.tensor([[2], [1]]),
        "response_length": torch.tensor([[3], [2]])}, forward_only=True)
    assert out.squeeze(-1).tolist() == [[1.0, 2.0, 3.0], [6.0, 7.0, 0.0]]


def test_pad_process_reference_vectors(reference_vectors):
    """remove_padding_and_split_to_list and pad_multiple (tests/ut/utils/test_pad_process.py:18-46), the
    TensorDict round trip by construction, get_last_reward against its closed form."""
    v = reference_vectors["remove_padding_and_split_to_list"]
    out = packing.remove_padding_and_split_to_list(torch.tensor(v["responses"]), v["eos_token_id"], v["pad_token_id"])
    assert [o.tolist() for o in out] == v["expected"]
    # pad token == eos token: the first pad token is kept; to_list drops the last token
    out = packing.remove_padding_and_split_to_list(torch.tensor(v["responses"]), 0, 0)
    assert [o.tolist() for o in out] == [[1, 2, 3, 4, 0], [4, 5, 6, 1, 1, 0]]
    assert packing.remove_padding_and_split_to_list(torch.tensor(v["responses"]), 0, 0, to_list=True) == \
        [[1, 2, 3, 4], [4, 5, 6, 1, 1]]
    m = reference_vectors["pad_multiple"]
    got = packing.pad_multiple([torch.tensor(x) for x in m["data_list"]], m["pad_id"], m["multiple"])
    assert got.tolist() == m["expected"]
    cols = {"a": [torch.tensor([1, 2, 3]), torch.tensor([4])], "b": [torch.tensor([5.0]), torch.tensor([6.0, 7.0])]}
    packed = packing.padding_dict_to_tensor_dict(cols)
    assert packed["a"].tolist() == [[1, 2, 3], [4, 0, 0]] and packed["b"].tolist() == [[5.0, 0.0], [6.0, 7.0]]
    assert packed["original_length"].tolist() == [3, 1, 1, 2]
    back = packing.remove_padding_tensor_dict_to_dict(packed)
    for k in cols:
        assert [r.tolist() for r in back[k]] == [c.tolist() for c in cols[k]]
    assert packing.remove_padding_tensor_dict_to_dict(None) == {}
    r = torch.tensor([[1.0], [3.0], [2.0], [2.0]])
    got = advantage.get_last_reward(r, 2)
    assert torch.allclose(got, torch.tensor([[-0.70710677], [0.70710677], [0.0], [0.0]]), atol=1e-6)


def test_oracle_reproduces_its_golden_vectors(oracle_vectors):
    """tests/golden/oracle_vectors.json was written by tests/golden/make_oracle_vectors.py from this
    repository's oracle; replaying the script must give the same numbers (drift guard)."""
    import importlib.util
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_oracle_vectors.py")
    spec = importlib.util.spec_from_file_location("make_oracle_vectors", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()

    def close(a, b, where):
        if isinstance(a, dict):
            assert set(a) == set(b), where
            for k in a:
                close(a[k], b[k], where + "/" + k)
        elif isinstance(a, list):
            assert len(a) == len(b), where
            for i, (x, y) in enumerate(zip(a, b)):
                close(x, y, where + "[%d]" % i)
        elif isinstance(a, float):
            assert a == pytest.approx(b, rel=1e-6, abs=1e-9), where
        else:
            assert a == b, where

    close(fresh, oracle_vectors, "")


def test_pack_maps_property_based():
    """Random ragged batches: packing then unpacking returns every valid position, padded sequence
    starts are multiples of the alignment, and the index maps agree with a direct restatement."""
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=60, deadline=None)
    @given(st.lists(st.tuples(st.integers(1, 5), st.integers(0, 9)), min_size=1, max_size=6),
           st.sampled_from([1, 2, 4, 8]), st.integers(0, 10 ** 6))
    def check(lengths, align, seed):
        gen = torch.Generator().manual_seed(seed)
        batch = len(lengths)
        plen = torch.tensor([[p] for p, _ in lengths], dtype=torch.int32)
        rlen = torch.tensor([[r] for _, r in lengths], dtype=torch.int32)
        width = int((plen + rlen).max())
        ids = torch.randint(1, 1000, (batch, width), generator=gen)
        mask = packing.generate_mask(ids, plen + rlen)
        ids = ids * mask
        p_ids, p_pos, _, seqlens, cu = packing.preprocess_packed_seqs(ids, ids, mask, align)
        assert seqlens.tolist() == (plen + rlen).flatten().tolist()
        assert all(int(c) % align == 0 for c in cu) and int(cu[-1]) == p_ids.shape[1]
        for i in range(batch):
            n, lo = int(seqlens[i]), int(cu[i])
            assert p_ids[0, lo:lo + n].tolist() == ids[i, :n].tolist()
            assert p_pos[0, lo:lo + n].tolist() == list(range(n))
            assert not p_ids[0, lo + n:int(cu[i + 1])].any()
        back = packing.postprocess_packed_seqs(p_ids.float(), seqlens, cu, width)
        assert torch.equal(back.long() * mask, ids)
        resp_w = max(int(rlen.max()), 1)
        cut = packing.postprocess_packed_seqs(p_ids.float(), seqlens, cu, resp_w, prompt_length=plen)
        for i in range(batch):
            p, r = int(plen[i]), int(rlen[i])
            want = ids[i, p - 1:p - 1 + r].tolist()
            assert cut[i, :r].long().tolist() == want

    check()
