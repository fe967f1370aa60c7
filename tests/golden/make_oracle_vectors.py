"""Writes tests/golden/oracle_vectors.json: seeded inputs and the outputs of THIS repository's oracle
for every kernel family at tiny shapes.  The file guards the oracle against drift (a CPU test replays
it) and gives the GPU tests fixed vectors next to the randomised ones.  Nothing from the reference is
imported or run; run from the repository root:  python tests/golden/make_oracle_vectors.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import advantage, loss, packing, vocab  # noqa: E402


def lst(t):
    return t.detach().tolist()


def build():
    gen = torch.Generator().manual_seed(20250)
    out = {}
    # K1-K3: log-prob, entropy and their gradient
    z = (torch.randn(6, 40, generator=gen) * 2).to(torch.bfloat16).float()      # bf16-representable
    y = torch.randint(0, 40, (6,), generator=gen)
    g_lp = torch.randn(6, generator=gen) * 0.1
    g_h = torch.randn(6, generator=gen) * 0.01
    zr = z.clone().requires_grad_()
    lp = vocab.compute_log_probs(zr, y)
    ent = vocab.vocab_parallel_entropy(zr)
    (dz,) = torch.autograd.grad((lp * g_lp).sum() + (ent * g_h).sum(), zr)
    out["vocab"] = {"logits": lst(z), "labels": lst(y), "g_logp": lst(g_lp), "g_entropy": lst(g_h),
                    "logp": lst(lp), "entropy": lst(ent), "dlogits": lst(dz)}
    # K4-K6: packing index maps
    plen = torch.tensor([[2], [1], [3], [1]], dtype=torch.int32)
    rlen = torch.tensor([[3], [5], [0], [2]], dtype=torch.int32)
    width = 9
    ids = torch.randint(1, 50, (4, width), generator=gen)
    mask1d = packing.generate_mask(ids, plen + rlen)
    ids = ids * mask1d
    labels = torch.cat([ids[:, 1:], torch.zeros(4, 1, dtype=ids.dtype)], 1)
    packs = {}
    for align in (1, 4):
        p_ids, p_pos, p_lab, seqlens, cu = packing.preprocess_packed_seqs(ids, labels, mask1d, align)
        per_row = torch.arange(p_ids.shape[1], dtype=torch.float32).unsqueeze(0)
        packs[str(align)] = {"ids": lst(p_ids), "position_ids": lst(p_pos), "labels": lst(p_lab), "seqlens": lst(seqlens),
                             "cu_seqlens_padded": lst(cu),
                             "unpacked_rows": lst(packing.postprocess_packed_seqs(per_row, seqlens, cu, 5, prompt_length=plen))}
    out["packing"] = {"input_ids": lst(ids), "labels": lst(labels), "attention_mask": lst(mask1d), "prompt_length": lst(plen),
                      "response_length": lst(rlen), "by_alignment": packs}
    # K7: group-relative advantages
    rewards = torch.tensor([[1.0], [0.0], [0.0], [1.0], [0.5], [0.25], [2.0], [2.0]])
    rl = torch.tensor([[3], [1], [2], [3], [3], [2], [1], [3]])
    mask = packing.generate_mask(torch.zeros(8, 3), rl)
    adv, _ = advantage.compute_group_norm_advantage_return(rewards, mask, rl, 4)
    out["advantage"] = {"rewards": lst(rewards), "response_length": lst(rl), "group": 4, "advantages": lst(adv)}
    # K8: policy losses on [B, L] operands, with the gradient with respect to log_prob
    B, L = 4, 5
    lp = -torch.rand(B, L, generator=gen) * 3
    old = lp + torch.randn(B, L, generator=gen) * 0.3
    ref = lp + torch.randn(B, L, generator=gen) * 0.3
    advs = torch.randn(B, 1, generator=gen).repeat(1, L)
    ent = torch.rand(B, L, generator=gen) * 2
    m = packing.generate_mask(lp, torch.tensor([[5], [2], [4], [1]])).float()
    cases = {}
    lpr = lp.clone().requires_grad_()
    res = loss.grpo_policy_loss(old, lpr, ref, advs, ent, m, 0.2, 0.01, "low_var_kl", 0.003)
    (g,) = torch.autograd.grad(res[0], lpr)
    cases["grpo"] = {"outputs": [float(x.detach()) for x in res], "g_log_prob": lst(g)}
    for token_level in (True, False):
        lpr = lp.clone().requires_grad_()
        res = loss.dapo_policy_loss(old, lpr, ent, 0.003, advs, m, 0.2, 0.28, token_level)
        (g,) = torch.autograd.grad(res[0], lpr)
        cases["dapo_token" if token_level else "dapo_seq"] = {"outputs": [float(x.detach()) for x in res], "g_log_prob": lst(g)}
    out["policy_loss"] = {"log_prob": lst(lp), "old_log_prob": lst(old), "ref_log_prob": lst(ref), "advantages": lst(advs),
                          "entropy": lst(ent), "mask": lst(m), "cases": cases}
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_vectors.json")
    with open(path, "w") as f:
        json.dump(build(), f, indent=1)
    print("wrote", path)
