"""GPU parity tests: every HIP entry point, called through the C ABI (ctypes) by the package's
host code, against the CPU oracle on the same seeded inputs.

Tolerances (fp32 accumulate against the oracle's fp32 up-cast): index maps, masks and group
assignment bit-exact; logp / entropy / advantages 1e-3 abs; loss 1e-4 rel; dlogits 2e-3 abs.
The observed errors are far smaller; tighter bounds are asserted where the arithmetic allows.
"""
import math
import os
import random

import numpy as np
import pytest
import torch

import mindspeed_rl_amd as mrl
from mindspeed_rl_amd import _lib
from oracle import advantage as o_adv
from oracle import loss as o_loss
from oracle import packing as o_pack
from oracle import vocab as o_vocab

pytestmark = pytest.mark.gpu

TOL_LOGP = 1e-3
TOL_DLOGITS = 2e-3
TOL_LOSS_REL = 1e-4


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    _lib.load()
    return torch.device("cuda:0")


def _logits(gen, rows, vocab, dtype, scale=3.0):
    return (torch.randn(rows, vocab, generator=gen) * scale).to(dtype)


def test_against_committed_oracle_vectors(dev, oracle_vectors):
    """Fixed vectors (tests/golden/oracle_vectors.json, written by this repository's oracle) through the
    HIP path: sweeps, index maps, advantages and the [B, L] policy losses."""
    v = oracle_vectors["vocab"]
    for dtype in (torch.float32, torch.bfloat16):
        z = torch.tensor(v["logits"]).to(dtype).to(dev).requires_grad_()          # the logits are bf16-representable
        lp, h, _ = mrl.vocab_logprob_entropy(z, torch.tensor(v["labels"]).to(dev))
        assert (lp.cpu() - torch.tensor(v["logp"])).abs().max().item() < 1e-5
        assert (h.cpu() - torch.tensor(v["entropy"])).abs().max().item() < 1e-5
        (dz,) = torch.autograd.grad([lp, h], z, [torch.tensor(v["g_logp"]).to(dev), torch.tensor(v["g_entropy"]).to(dev)])
        tol = 1e-6 if dtype == torch.float32 else TOL_DLOGITS
        assert (dz.float().cpu() - torch.tensor(v["dlogits"])).abs().max().item() < tol
    pk = oracle_vectors["packing"]
    ids, labels = torch.tensor(pk["input_ids"]).to(dev), torch.tensor(pk["labels"]).to(dev)
    mask = torch.tensor(pk["attention_mask"]).to(dev)
    plen = torch.tensor(pk["prompt_length"], dtype=torch.int32).to(dev)
    for align, want in pk["by_alignment"].items():
        p_ids, p_pos, p_lab, seqlens, cu = mrl.preprocess_packed_seqs(ids, labels, mask, int(align))
        assert p_ids.cpu().tolist() == want["ids"] and p_pos.cpu().tolist() == want["position_ids"]
        assert p_lab.cpu().tolist() == want["labels"] and seqlens.cpu().tolist() == want["seqlens"]
        assert cu.cpu().tolist() == want["cu_seqlens_padded"]
        rows = torch.arange(p_ids.shape[1], dtype=torch.float32, device=dev).unsqueeze(0)
        got = mrl.postprocess_packed_seqs(rows, seqlens, cu, 5, prompt_length=plen)
        assert got.cpu().tolist() == want["unpacked_rows"]
    a = oracle_vectors["advantage"]
    rl = torch.tensor(a["response_length"]).to(dev)
    m = mrl.generate_mask(torch.zeros(8, 3, device=dev), rl)
    adv, _ = mrl.compute_group_norm_advantage_return(torch.tensor(a["rewards"]).to(dev), m, rl, a["group"])
    assert (adv.cpu() - torch.tensor(a["advantages"])).abs().max().item() < 1e-6
    pl = oracle_vectors["policy_loss"]
    t = {k: torch.tensor(pl[k]).to(dev) for k in ("log_prob", "old_log_prob", "ref_log_prob", "advantages", "entropy", "mask")}
    runs = {"grpo": dict(ref_log_prob=t["ref_log_prob"], clip_low=0.2, clip_high=0.2, kl_penalty="low_var_kl", kl_coef=0.01,
                         entropy_coeff=0.003, token_level_loss=True),
            "dapo_token": dict(ref_log_prob=None, clip_low=0.2, clip_high=0.28, entropy_coeff=0.003, token_level_loss=True),
            "dapo_seq": dict(ref_log_prob=None, clip_low=0.2, clip_high=0.28, entropy_coeff=0.003, token_level_loss=False)}
    for name, kwargs in runs.items():
        want = pl["cases"][name]
        lp = t["log_prob"].clone().requires_grad_()
        ref = kwargs.pop("ref_log_prob")
        loss, out = mrl.policy_loss(lp, t["entropy"], t["old_log_prob"], ref, t["advantages"], mask=t["mask"], **kwargs)
        assert loss.item() == pytest.approx(want["outputs"][0], rel=TOL_LOSS_REL, abs=1e-7), name
        (g,) = torch.autograd.grad(loss, lp)
        assert (g.cpu() - torch.tensor(want["g_log_prob"])).abs().max().item() < 1e-6, name


# --------------------------------------------------------------------------------- vocab sweep
@pytest.mark.parametrize("dtype,vocab,rows", [
    (torch.float32, 32000, 64), (torch.bfloat16, 152064, 24), (torch.bfloat16, 129280, 16),
    (torch.float16, 32000, 32), (torch.float32, 501, 37), (torch.bfloat16, 1003, 19),
    (torch.bfloat16, 7, 5), (torch.float32, 3, 4), (torch.bfloat16, 8200, 9),
])
@pytest.mark.parametrize("label_dtype", [torch.int64, torch.int32])
def test_vocab_forward_backward_parity(dev, dtype, vocab, rows, label_dtype):
    gen = torch.Generator().manual_seed(vocab * 7 + rows)
    z = _logits(gen, rows, vocab, dtype)
    y = torch.randint(0, vocab, (rows,), generator=gen).to(label_dtype)
    # incoming gradients of realistic size (|A|/N in training is far smaller still): a bf16 dlogit
    # carries 2^-9 relative rounding, so the absolute tolerance presumes |dlogit| < 1
    g_lp = torch.randn(rows, generator=gen) * 0.1
    g_h = torch.randn(rows, generator=gen) * 0.01
    g_lp[0] = 0.0
    g_h[0] = 0.0                                        # a dead row: zeros without reading
    # oracle on the fp32 up-cast
    zo = z.float().requires_grad_()
    lp_o = o_vocab.compute_log_probs(zo, y.long())
    h_o = o_vocab.vocab_parallel_entropy(zo)
    (dz_o,) = torch.autograd.grad((lp_o * g_lp).sum() + (h_o * g_h).sum(), zo)
    lp64, h64, lse64 = o_vocab.logprob_entropy_fp64(z, y)

    zd = z.to(dev).requires_grad_()
    lp, h, lse = mrl.vocab_logprob_entropy(zd, y.to(dev))
    assert lp.dtype == torch.float32 and lp.shape == (rows,)
    assert (lp.cpu() - lp_o.detach()).abs().max().item() < TOL_LOGP
    assert (h.cpu() - h_o.detach()).abs().max().item() < TOL_LOGP
    # against fp64 the kernel is as good as the fp32 torch chain
    assert (lp.cpu().double() - lp64).abs().max().item() < 2e-5
    assert (h.cpu().double() - h64).abs().max().item() < 5e-5
    assert (lse.cpu().double() - lse64).abs().max().item() < 2e-5
    (dz,) = torch.autograd.grad([lp, h], zd, [g_lp.to(dev), g_h.to(dev)])
    assert dz.dtype == dtype and dz.shape == z.shape
    assert (dz.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    assert torch.equal(dz[0].cpu(), torch.zeros(vocab, dtype=dtype))
    assert torch.equal(zd.detach().cpu(), z), "the sweep must not write its input"


def test_vocab_entropy_skipped_and_separate_functions(dev):
    gen = torch.Generator().manual_seed(5)
    z = _logits(gen, 33, 4096, torch.bfloat16)
    y = torch.randint(0, 4096, (1, 33), generator=gen)
    zd = z.to(dev).unsqueeze(0).requires_grad_()
    lp = mrl.compute_log_probs(zd, y.to(dev))
    assert lp.shape == (1, 33)
    lp_o = o_vocab.compute_log_probs(z.float().unsqueeze(0), y)
    assert (lp.detach().cpu() - lp_o).abs().max().item() < 1e-4
    ent = mrl.vocab_parallel_entropy(zd)
    assert (ent.detach().cpu() - o_vocab.vocab_parallel_entropy(z.float().unsqueeze(0))).abs().max().item() < 1e-4
    ce = mrl.vocab_parallel_cross_entropy(vocab_parallel_logits=zd, target=y.to(dev))
    assert torch.equal(ce, -lp)
    # gradient of logp alone (no entropy term compiled in)
    g = torch.randn(1, 33, generator=gen) * 0.1
    (dz,) = torch.autograd.grad(lp, zd, g.to(dev))
    zo = z.float().unsqueeze(0).requires_grad_()
    (dz_o,) = torch.autograd.grad(o_vocab.compute_log_probs(zo, y), zo, g)
    assert (dz.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    # an injected cross entropy is honoured (the reference's hook)
    calls = []

    def fake_ce(vocab_parallel_logits, target):
        calls.append(1)
        return torch.zeros(target.shape, device=target.device)

    mrl.set_vocab_parallel(fake_ce)
    try:
        assert mrl.compute_log_probs(zd, y.to(dev)).abs().sum().item() == 0 and calls
    finally:
        mrl.set_vocab_parallel(None)


def test_vocab_out_of_range_labels_temperature_and_row_mask(dev):
    gen = torch.Generator().manual_seed(6)
    z = _logits(gen, 12, 2048, torch.float32, scale=4.0)
    y = torch.randint(0, 2048, (12,), generator=gen)
    y[3] = -1
    y[7] = 2048
    temp = 0.7
    zo = (z / temp).requires_grad_()
    lp_o = o_vocab.compute_log_probs(zo, y)
    h_o = o_vocab.vocab_parallel_entropy(zo)
    g = torch.randn(12, generator=gen)
    (dz_o,) = torch.autograd.grad((lp_o * g).sum() + (h_o * 0.3).sum(), zo)
    dz_o = dz_o / temp                                  # autograd of output.div_(temperature)
    active = torch.ones(12, dtype=torch.bool)
    active[5] = False
    zd = z.to(dev).requires_grad_()
    lp, h, _ = mrl.vocab_logprob_entropy(zd, y.to(dev), inv_temperature=1.0 / temp, row_active=active.to(dev))
    keep = active.clone()
    assert (lp.cpu()[keep] - lp_o.detach()[keep]).abs().max().item() < 1e-4
    assert (h.cpu()[keep] - h_o.detach()[keep]).abs().max().item() < 1e-4
    assert lp[5].item() == 0.0 and h[5].item() == 0.0
    gd = g.clone()
    gd[5] = 0.0
    gh = torch.full((12,), 0.3)
    gh[5] = 0.0
    (dz,) = torch.autograd.grad([lp, h], zd, [gd.to(dev), gh.to(dev)])
    dz_o[5] = 0.0
    assert (dz.cpu() - dz_o).abs().max().item() < 1e-4


def test_vocab_strided_rows_inplace_and_fp32_grad(dev):
    gen = torch.Generator().manual_seed(8)
    rows, vocab, stride = 10, 1000, 1024
    buf = torch.zeros(rows, stride, dtype=torch.bfloat16)
    buf[:, :vocab] = _logits(gen, rows, vocab, torch.bfloat16)
    y = torch.randint(0, vocab, (rows,), generator=gen)
    g = torch.randn(rows, generator=gen) * 0.1
    zo = buf[:, :vocab].float().requires_grad_()
    lp_o = o_vocab.compute_log_probs(zo, y)
    (dz_o,) = torch.autograd.grad(lp_o, zo, g)
    bd = buf.to(dev)
    view = bd[:, :vocab]
    lp = torch.empty(rows, device=dev)
    lse = torch.empty(rows, device=dev)
    s = _lib.stream(dev)
    yd = y.to(dev)
    _lib.call("mrl_vocab_logprob_fwd", view.data_ptr(), _lib.BF16, rows, vocab, stride, yd.data_ptr(), _lib.I64, None,
              1.0, lp.data_ptr(), None, lse.data_ptr(), s)
    assert (lp.cpu() - lp_o.detach()).abs().max().item() < 1e-4
    gd = g.to(dev)
    # fp32 gradient from bf16 logits, separate buffer with its own stride
    d32 = torch.full((rows, 1000), 7.0, device=dev)
    _lib.call("mrl_vocab_logprob_bwd", view.data_ptr(), _lib.BF16, rows, vocab, stride, yd.data_ptr(), _lib.I64, 1.0,
              lse.data_ptr(), None, gd.data_ptr(), None, d32.data_ptr(), _lib.F32, 1000, s)
    assert (d32.cpu() - dz_o).abs().max().item() < 1e-5
    # in-place: dlogits overwrite the logits, padding columns stay untouched
    bd[:, vocab:] = 5.0
    _lib.call("mrl_vocab_logprob_bwd", view.data_ptr(), _lib.BF16, rows, vocab, stride, yd.data_ptr(), _lib.I64, 1.0,
              lse.data_ptr(), None, gd.data_ptr(), None, view.data_ptr(), _lib.BF16, stride, s)
    torch.cuda.synchronize()
    assert (bd[:, :vocab].float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    assert (bd[:, vocab:] == 5.0).all().item()
    # misaligned base pointer (odd element offset): scalar head/tail path and the scalar backward
    flat = torch.zeros(rows * 1001 + 3, dtype=torch.bfloat16, device=dev)
    odd = flat[3:].view(rows, 1001)[:, :1000]
    odd.copy_(buf[:, :vocab].to(dev))
    lp2 = torch.empty(rows, device=dev)
    _lib.call("mrl_vocab_logprob_fwd", odd.data_ptr(), _lib.BF16, rows, vocab, 1001, yd.data_ptr(), _lib.I64, None, 1.0,
              lp2.data_ptr(), None, lse.data_ptr(), s)
    assert torch.allclose(lp2, lp, atol=1e-6)
    dodd = torch.empty(rows, 1000, dtype=torch.bfloat16, device=dev)
    _lib.call("mrl_vocab_logprob_bwd", odd.data_ptr(), _lib.BF16, rows, vocab, 1001, yd.data_ptr(), _lib.I64, 1.0,
              lse.data_ptr(), None, gd.data_ptr(), None, dodd.data_ptr(), _lib.BF16, 1000, s)
    assert (dodd.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS


def test_vocab_properties_at_full_vocab(dev):
    """Size-independent properties at the Qwen2.5 vocabulary (152064, bf16), generated on the device."""
    torch.manual_seed(11)
    rows, vocab = 512, 152064
    z = (torch.randn(rows, vocab, device=dev) * 3).to(torch.bfloat16)
    y = torch.randint(0, vocab, (rows,), device=dev)
    zr = z.requires_grad_()
    lp, h, lse = mrl.vocab_logprob_entropy(zr, y)
    # against torch on the device in fp32 (a second, independent implementation)
    ref = torch.log_softmax(z.float(), -1)
    assert (lp - ref.gather(-1, y[:, None]).squeeze(-1)).abs().max().item() < 1e-4
    ent_ref = -(ref.exp() * ref).sum(-1)
    assert (h - ent_ref).abs().max().item() < 2e-4
    assert ((h >= 0) & (h <= math.log(vocab) + 1e-4)).all().item()
    # shift invariance, on logits quantised to multiples of 1/8 in [-8, 8] so that adding 8 is exact in bf16
    zq = (torch.round(z.detach().float().clamp(-8, 8) * 8) / 8).to(torch.bfloat16)
    zq8 = (zq.float() + 8.0).to(torch.bfloat16)
    assert torch.equal(zq8.float() - 8.0, zq.float())
    lp1, h1, lse1 = mrl.vocab_logprob_entropy(zq, y)
    lp2, h2, lse2 = mrl.vocab_logprob_entropy(zq8, y)
    assert (lp2 - lp1).abs().max().item() < 1e-4 and (h2 - h1).abs().max().item() < 2e-4
    assert (lse2 - lse1 - 8.0).abs().max().item() < 1e-4
    # every row of dlogits sums to ~0 (softmax gradients are tangent to the simplex)
    g_lp = torch.randn(rows, device=dev) * 0.1
    g_h = torch.randn(rows, device=dev) * 0.01
    (dz,) = torch.autograd.grad([lp, h], zr, [g_lp, g_h])
    assert dz.float().sum(-1).abs().max().item() < 2e-2          # bf16 rounding of 152064 terms
    closed = g_lp[:, None] * (torch.nn.functional.one_hot(y, vocab) - ref.exp()) \
        - g_h[:, None] * ref.exp() * (z.detach().float() - (ref.exp() * z.detach().float()).sum(-1, keepdim=True))
    assert (dz.float() - closed).abs().max().item() < TOL_DLOGITS
    # linearity in the incoming gradient
    (dz2,) = torch.autograd.grad([mrl.vocab_logprob_entropy(zr, y)[0]], zr, [2.0 * g_lp])
    (dz1,) = torch.autograd.grad([mrl.vocab_logprob_entropy(zr, y)[0]], zr, [g_lp])
    assert (dz2.float() - 2 * dz1.float()).abs().max().item() < 2e-3


# --------------------------------------------------------------------------------- index maps
def _random_lengths(gen, batch, width, max_prompt=6):
    plen = torch.randint(1, max_prompt, (batch, 1), generator=gen, dtype=torch.int32)
    rlen = torch.randint(0, width - max_prompt, (batch, 1), generator=gen, dtype=torch.int32)
    return plen, rlen


@pytest.mark.parametrize("align", [1, 2, 8, 16])
@pytest.mark.parametrize("id_dtype", [torch.int64, torch.int32])
def test_pack_unpack_bit_exact(dev, align, id_dtype):
    gen = torch.Generator().manual_seed(100 + align)
    batch, width, resp_w = 37, 96, 90
    plen, rlen = _random_lengths(gen, batch, width)
    rlen[4] = 0
    rlen[5] = 0                                          # empty responses, back to back
    ids = torch.randint(1, 50000, (batch, width), generator=gen).to(id_dtype)
    labels = torch.cat([ids[:, 1:], torch.zeros(batch, 1, dtype=id_dtype)], 1)
    mask_o = o_pack.generate_mask(ids, plen + rlen)
    mask = mrl.generate_mask(ids.to(dev), (plen + rlen).to(dev))
    assert mask.dtype == torch.int64 and torch.equal(mask.cpu(), mask_o)
    want = o_pack.preprocess_packed_seqs(ids, labels, mask_o, align)
    got = mrl.preprocess_packed_seqs(ids.to(dev), labels.to(dev), mask, align)
    for a, b in zip(got, want):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.equal(a.cpu(), b)
    _, _, _, seqlens, cu = got
    # unpack, with and without the prompt shift, fp32 and int payloads, and a trailing dimension
    packed = torch.randn(1, want[0].shape[1], generator=gen)
    for prompt in (None, plen):
        w = o_pack.postprocess_packed_seqs(packed, want[3], want[4], resp_w if prompt is not None else width, prompt)
        g = mrl.postprocess_packed_seqs(packed.to(dev), seqlens, cu, resp_w if prompt is not None else width,
                                        None if prompt is None else prompt.to(dev))
        assert torch.equal(g.cpu(), w)
    back = mrl.postprocess_packed_seqs(got[0], seqlens, cu, width)
    assert torch.equal(back.cpu(), ids * mask_o.to(id_dtype))
    p3 = torch.randn(1, want[0].shape[1], 5, generator=gen).to(torch.bfloat16)
    w3 = o_pack.postprocess_packed_seqs(p3, want[3], want[4], resp_w, plen)
    g3 = mrl.postprocess_packed_seqs(p3.to(dev), seqlens, cu, resp_w, plen.to(dev))
    assert torch.equal(g3.cpu(), w3)
    # adjoint: <unpack(x), g> == <x, scatter(g)>, and the scatter equals autograd of the oracle
    x = packed.clone().requires_grad_()
    go = torch.randn(batch, resp_w, generator=gen)
    (gx_o,) = torch.autograd.grad(o_pack.postprocess_packed_seqs(x, want[3], want[4], resp_w, plen), x, go)
    xd = packed.to(dev).requires_grad_()
    (gx,) = torch.autograd.grad(mrl.postprocess_packed_seqs(xd, seqlens, cu, resp_w, plen.to(dev)), xd, go.to(dev))
    assert torch.equal(gx.cpu(), gx_o)


def test_pack_index_edge_cases(dev):
    # empty batch row, all-zero mask rows, float and bool masks, int32 lengths
    mask = torch.tensor([[1, 1, 1, 0], [0, 0, 0, 0], [1, 0, 0, 0], [1, 1, 1, 1]])
    for cast in (torch.int64, torch.int32, torch.bool, torch.float32):
        seqlens, cu, total = mrl.pack_index(mask.to(cast).to(dev), 4)
        assert seqlens.tolist() == [3, 0, 1, 4] and cu.tolist() == [0, 4, 4, 8, 12] and total.item() == 12
    ids = torch.arange(16).view(4, 4)
    got = mrl.preprocess_packed_seqs(ids.to(dev), ids.to(dev), mask.to(dev), 4)
    want = o_pack.preprocess_packed_seqs(ids, ids, mask, 4)
    for a, b in zip(got, want):
        assert torch.equal(a.cpu(), b)
    # a batch larger than one scan chunk (1024) with ragged lengths
    gen = torch.Generator().manual_seed(3)
    lens = torch.randint(0, 50, (2500,), generator=gen, dtype=torch.int32)
    big = o_pack.generate_mask(torch.zeros(2500, 50), lens)
    seqlens, cu, total = mrl.pack_index(big.to(dev), 8)
    padded = (lens + 7) // 8 * 8
    assert torch.equal(seqlens.cpu(), lens)
    assert cu.cpu().tolist() == [0] + torch.cumsum(padded, 0).tolist()
    assert total.item() == int(padded.sum())


def test_padded_window_bit_exact(dev, reference_vectors):
    v = reference_vectors["truncate_middle_and_pad"]
    out = mrl.truncate_middle_and_pad(torch.tensor(v["responses"]).to(dev), torch.tensor(v["input_tensor"]).to(dev),
                                      torch.tensor(v["truncate_lengths"]).to(dev), v["pad_value"])
    assert torch.equal(out.cpu(), torch.tensor(v["expected"]))
    v = reference_vectors["generate_mask"]
    m = mrl.generate_mask(torch.tensor(v["data_pad"]).to(dev), torch.tensor(v["seq_lengths"]).to(dev))
    assert m.cpu().tolist() == v["expected"]
    gen = torch.Generator().manual_seed(21)
    batch, width, resp_w = 23, 70, 64
    plen, rlen = _random_lengths(gen, batch, width)
    window = o_pack.response_window(plen, rlen)
    assert torch.equal(mrl.response_window(plen.to(dev), rlen.to(dev)).cpu(), window)
    resp = torch.zeros(batch, resp_w)
    vals = torch.randn(batch, width, generator=gen)
    for pad in (0.0, -1.5):
        want = o_pack.truncate_prompt_and_pad(resp, vals, window, pad)
        got = mrl.truncate_prompt_and_pad(resp.to(dev), vals.to(dev), window.to(dev), pad)
        assert torch.equal(got.cpu(), want)
    v3 = torch.randn(batch, width, 6, generator=gen).to(torch.bfloat16)
    assert torch.equal(mrl.truncate_middle_and_pad(resp.to(dev), v3.to(dev), window.to(dev)).cpu(),
                       o_pack.truncate_middle_and_pad(resp, v3, window))
    # windows that leave [0, width] are clamped like torch.clamp does
    wild = window.clone()
    wild[0] = torch.tensor([-3, 5])
    wild[1] = torch.tensor([60, 200])
    assert torch.equal(mrl.truncate_prompt_and_pad(resp.to(dev), vals.to(dev), wild.to(dev)).cpu(),
                       o_pack.truncate_prompt_and_pad(resp, vals, wild))
    x = vals.clone().requires_grad_()
    go = torch.randn(batch, resp_w, generator=gen)
    (gx_o,) = torch.autograd.grad(o_pack.truncate_prompt_and_pad(resp, x, window), x, go)
    xd = vals.to(dev).requires_grad_()
    (gx,) = torch.autograd.grad(mrl.truncate_prompt_and_pad(resp.to(dev), xd, window.to(dev)), xd, go.to(dev))
    assert torch.equal(gx.cpu(), gx_o)


def test_wire_format_bit_exact(dev):
    """unpack_pad_experience and truncate_rows against the reference's loops (oracle), bit for bit."""
    gen = torch.Generator().manual_seed(61)
    batch = 37
    lens_a = torch.randint(0, 50, (batch,), generator=gen, dtype=torch.int32)
    lens_b = torch.randint(1, 9, (batch,), generator=gen, dtype=torch.int32)
    data = {"responses": torch.randint(0, 1000, (int(lens_a.sum()),), generator=gen),
            "old_log_prob": torch.randn(int(lens_a.sum()), generator=gen),
            "position_ids": torch.randint(0, 99, (3, int(lens_b.sum())), generator=gen),
            "response_length": lens_a.clone()}
    lens = {"responses": lens_a, "old_log_prob": lens_a, "position_ids": lens_b, "response_length": torch.ones(batch, dtype=torch.int32)}
    for multiple in (1, 8):
        want = o_pack.unpack_pad_experience(data, lens, -7, multiple)
        got = mrl.unpack_pad_experience({k: v.to(dev) for k, v in data.items()}, lens, -7, multiple)
        assert set(got) == set(want)
        for k in want:
            assert got[k].dtype == want[k].dtype and got[k].shape == want[k].shape, k
            assert torch.equal(got[k].cpu(), want[k]), k
    with pytest.raises(ValueError):
        mrl.unpack_pad_experience({}, {}, 0, 1)
    tensor = torch.randint(0, 500, (batch, 40), generator=gen)
    tensor[3, 0] = -1
    tensor[4, 0] = -1
    idx = torch.randint(0, 41, (batch, 1), generator=gen)
    idx[3] = 0
    idx[5] = 0
    for left in (False, True):
        for cast in (torch.int64, torch.int32):
            want = o_pack.truncate_rows(tensor.to(cast), idx, left)
            got = mrl.truncate_rows(tensor.to(cast).to(dev), idx.to(dev), left)
            assert len(got) == len(want)
            for a, b in zip(got, want):
                assert a.dtype == b.dtype and torch.equal(a, b)
    f = torch.randn(batch, 40, generator=gen)
    for left in (False, True):
        for a, b in zip(mrl.truncate_rows(f.to(dev), idx.to(dev), left), o_pack.truncate_rows(f, idx, left)):
            assert a.dtype == b.dtype and torch.equal(a, b)
    # packing: lists of samples (the reference's input) and padded columns + lengths (the device form)
    cu_a = torch.cat([torch.zeros(1, dtype=torch.int64), lens_a.long().cumsum(0)])
    cu_b = torch.cat([torch.zeros(1, dtype=torch.int64), lens_b.long().cumsum(0)])
    samples = {"responses": [data["responses"][cu_a[i]:cu_a[i + 1]] for i in range(batch)],
               "old_log_prob": [data["old_log_prob"][cu_a[i]:cu_a[i + 1]] for i in range(batch)],
               "position_ids": [data["position_ids"][:, cu_b[i]:cu_b[i + 1]] for i in range(batch)]}
    want, want_len = o_pack.pack_experience_columns("actor_train", samples, batch)
    got, got_len = mrl.pack_experience_columns("actor_train", {k: [t.to(dev) for t in v] for k, v in samples.items()},
                                               batch)
    for k in want:
        assert got[k].dtype == want[k].dtype and torch.equal(got[k].cpu(), want[k]), k
        assert got_len[k].dtype == torch.int32 and torch.equal(got_len[k].cpu(), want_len[k]), k
    padded = o_pack.unpack_pad_experience({k: data[k] for k in ("responses", "old_log_prob")},
                                          {k: lens[k] for k in ("responses", "old_log_prob")}, -7, 8)
    got, got_len = mrl.pack_padded_columns({k: v.to(dev) for k, v in padded.items()},
                                           {"responses": lens_a.to(dev), "old_log_prob": lens_a.view(-1, 1)})
    for k in padded:
        assert torch.equal(got[k].cpu(), data[k]) and torch.equal(got_len[k].cpu(), lens_a), k
    right = torch.flip(padded["responses"], dims=[1])          # the same samples, reversed and right-aligned
    got, _ = mrl.pack_padded_columns({"r": right.to(dev)}, {"r": lens_a}, left_pad=True)
    assert torch.equal(got["r"].cpu(), torch.cat([torch.flip(s_, dims=[0]) for s_ in samples["responses"]]))
    with pytest.raises(ValueError):
        mrl.pack_experience_columns("actor_train", {"responses": samples["responses"]}, batch - 1)


def test_pad_process_parity(dev, reference_vectors):
    """The rest of pad_process.py and the small helpers around the path, against the oracle."""
    v = reference_vectors["remove_padding_and_split_to_list"]
    out = mrl.remove_padding_and_split_to_list(torch.tensor(v["responses"]).to(dev), v["eos_token_id"], v["pad_token_id"])
    assert [o.tolist() for o in out] == v["expected"] and out[0].device.type == "cuda"
    m = reference_vectors["pad_multiple"]
    got = mrl.pad_multiple([torch.tensor(x).to(dev) for x in m["data_list"]], m["pad_id"], m["multiple"])
    assert got.tolist() == m["expected"]
    gen = torch.Generator().manual_seed(71)
    batch, width = 41, 130
    resp = torch.randint(1, 50, (batch, width), generator=gen)
    lens = torch.randint(0, width + 1, (batch,), generator=gen)
    lens[0], lens[1] = 0, width
    for i in range(batch):
        resp[i, int(lens[i]):] = 7
    resp[5, 3] = 7                                      # a pad token inside the response: the row is cut there
    for eos, pad in ((99, 7), (7, 7)):
        for cast in (torch.int64, torch.int32):
            for to_list in (False, True):
                want = o_pack.remove_padding_and_split_to_list(resp.to(cast), eos, pad, to_list)
                got = mrl.remove_padding_and_split_to_list(resp.to(cast).to(dev), eos, pad, to_list)
                assert len(got) == batch
                for a, b in zip(got, want):
                    if to_list:
                        assert a == b
                    else:
                        assert a.dtype == b.dtype and torch.equal(a.cpu(), b)
    cols = {"ids": [torch.randint(0, 9, (int(n),), generator=gen) for n in torch.randint(1, 20, (9,), generator=gen)],
            "lp": [torch.randn(int(n), generator=gen) for n in torch.randint(1, 33, (9,), generator=gen)]}
    want = o_pack.padding_dict_to_tensor_dict(cols)
    got = mrl.padding_dict_to_tensor_dict({k: [t.to(dev) for t in v_] for k, v_ in cols.items()})
    assert list(got) == list(want)
    for k in want:
        assert got[k].dtype == want[k].dtype and torch.equal(got[k].cpu(), want[k]), k
    back = mrl.remove_padding_tensor_dict_to_dict(got)
    for k in cols:
        assert all(torch.equal(a, b) for a, b in zip(back[k], cols[k]))
    assert mrl.remove_padding_tensor_dict_to_dict(None) == {}
    for k in (1, 2, 8):
        want = o_pack.pad_multiple(cols["lp"], 0.5, k)
        assert torch.equal(mrl.pad_multiple([t.to(dev) for t in cols["lp"]], 0.5, k).cpu(), want)
    # get_last_reward, clip_by_value, the reward model's loss object
    scores = torch.randn(24, 1, generator=gen)
    assert (mrl.get_last_reward(scores.to(dev), 8).cpu() - o_adv.get_last_reward(scores, 8)).abs().max().item() < 1e-5
    x = torch.randn(5, 6, generator=gen)
    assert torch.equal(mrl.clip_by_value(x.to(dev), torch.tensor(-0.5, device=dev), torch.tensor(0.25, device=dev)).cpu(),
                       torch.clamp(x, -0.5, 0.25))
    rw = mrl.LossFuncFactory.get_instance("ray_grpo", "reward")
    assert isinstance(rw, mrl.RewardLossFunc) and isinstance(mrl.LossFuncFactory.get_instance("ray_ppo", "reward"),
                                                                mrl.RewardLossFunc)
    seqlens = torch.tensor([3, 5], dtype=torch.int32)
    cu = torch.tensor([0, 4, 12], dtype=torch.int32)
    packed = torch.randn(1, 12, 1, generator=gen)
    got = rw.compute_loss(packed.to(dev), {}, forward_only=True, use_remove_padding=True, seqlens_in_batch=seqlens.to(dev),
                          cu_seqlens_padded=cu.to(dev), seq_len=6)
    assert torch.equal(got.cpu(), o_pack.postprocess_packed_seqs(packed, seqlens, cu, 6))
    plain = packed.to(dev)
    assert rw.compute_loss(plain, {}) is plain


# --------------------------------------------------------------------------------- PPO value side
def test_value_side_reference_vectors_on_device(dev, reference_vectors):
    w = reference_vectors["masked_whiten"]
    got = mrl.masked_whiten(torch.tensor(w["values"]).to(dev), torch.tensor(w["mask"]).to(dev))
    assert torch.allclose(got.cpu(), torch.tensor(w["expected"]), atol=w["atol"])
    v = reference_vectors["masked_var"]
    got = mrl.masked_var(torch.tensor(v["values"]).to(dev), torch.tensor(v["mask"]).to(dev), unbiased=True)
    assert torch.isclose(got.cpu(), torch.tensor(v["expected"]), atol=v["atol"])
    with pytest.raises(ValueError, match="At least one element"):
        mrl.masked_whiten(torch.ones(4, device=dev), torch.zeros(4, device=dev))
    g = reference_vectors["gae"]
    adv, ret = mrl.compute_gae_advantage_return(torch.tensor(g["token_level_rewards"]).to(dev),
                                                torch.tensor(g["values"]).to(dev), torch.tensor(g["eos_mask"]).to(dev),
                                                torch.tensor(g["gamma"]), torch.tensor(g["lam"]))
    assert torch.equal(adv.cpu(), torch.tensor(g["expected_advantages"]))
    assert torch.equal(ret.cpu(), torch.tensor(g["expected_returns"]))
    a = reference_vectors["adaptive_kl"]
    for case in a["cases"]:
        ctrl = mrl.AdaptiveKLController(a["init_kl_coef"], a["target_kl"], a["horizon"])
        ctrl.update(case["current_kl"], case["n_steps"])
        assert ctrl.value == case["expected"]
    crit = mrl.LossFuncFactory.get_instance(*reference_vectors["critic"]["registry_key"])
    assert isinstance(crit, mrl.CriticLossFunc)
    assert crit.cliprange_value == reference_vectors["critic"]["default_cliprange_value"]
    crit.add_loss_meta_info({"cliprange_value": 0.3})
    assert crit.cliprange_value == 0.3
    crit.add_loss_meta_info(None)
    c = reference_vectors["critic"]["no_clipping"]
    vf, frac = crit._compute_value_loss(torch.tensor(c["vpreds"]).to(dev), torch.tensor(c["returns"]).to(dev),
                                        torch.tensor(c["values"]).to(dev),
                                        torch.tensor(c["response_mask"], dtype=torch.float32).to(dev),
                                        c["cliprange_value"])
    assert frac.item() == 0 and vf.item() == 0.0
    with pytest.raises(ValueError, match="The responses is None"):
        crit._get_policy_loss_input({"values": torch.zeros(1, 1)})


@pytest.mark.parametrize("batch,width", [(37, 300), (3, 5000), (1, 1), (130, 2048)])
def test_gae_and_whitening_parity(dev, batch, width):
    """The scan is bit-identical to the reference's torch loop (same fp32 operation order), also across
    the 2048-entry staging chunks; the whitened advantages agree to fp32 summation-order accuracy."""
    gen = torch.Generator().manual_seed(batch * 100 + width)
    r = torch.randn(batch, width, generator=gen)
    v = torch.randn(batch, width, generator=gen)
    lens = torch.randint(1, width + 1, (batch, 1), generator=gen)
    mask = o_pack.generate_mask(r, lens)
    mask[0, 0] = 1
    if batch * width > 1:
        mask.view(-1)[1] = 1                # at least two entries: the unbiased variance is defined
    for gamma, lam in ((1.0, 0.95), (0.97, 0.9)):
        want_adv, want_ret = o_adv.compute_gae_advantage_return(r, v, mask, torch.tensor(gamma), torch.tensor(lam))
        adv, ret = mrl.compute_gae_advantage_return(r.to(dev), v.to(dev), mask.to(dev), gamma, lam)
        assert torch.equal(ret.cpu(), want_ret)
        scale = max(1.0, want_adv.abs().max().item())
        assert (adv.cpu() - want_adv).abs().max().item() < 1e-5 * scale
    # python floats, as the trainer passes them from its config: gamma * lam is formed in double and
    # rounded to fp32 once (for 0.9 * 0.95, 0.95 * 0.96 and 0.98 * 0.92 that differs from the product of
    # the two fp32-rounded factors by one unit in the last place)
    for gamma, lam in ((0.99, 0.95), (0.9, 0.95), (0.95, 0.96), (0.98, 0.92)):
        _, want_ret = o_adv.compute_gae_advantage_return(r, v, mask, gamma, lam)
        _, ret = mrl.compute_gae_advantage_return(r.to(dev), v.to(dev), mask.to(dev), gamma, lam)
        assert torch.equal(ret.cpu(), want_ret), (gamma, lam)
    # masked_var stand-alone, both estimators, float and bool masks
    for unbiased in (True, False):
        want = o_loss.masked_var(r, mask.float(), unbiased)
        for m in (mask.float(), mask.bool(), mask):
            got = mrl.masked_var(r.to(dev), m.to(dev), unbiased)
            assert got.item() == pytest.approx(want.item(), rel=1e-5, abs=1e-7)
    got = mrl.masked_whiten(r.to(dev), mask.to(dev), shift_mean=False)
    assert (got.cpu() - o_loss.masked_whiten(r, mask.float(), shift_mean=False)).abs().max().item() < 1e-5 * max(
        1.0, r.abs().max().item() * 2)


@pytest.mark.parametrize("penalty", ["kl", "abs", "mse", "low_var_kl"])
def test_kl_token_rewards_parity(dev, penalty):
    gen = torch.Generator().manual_seed(17)
    batch, width = 29, 77
    old = -torch.rand(batch, width, generator=gen) * 5
    ref = old + torch.randn(batch, width, generator=gen) * 0.3
    lens = torch.randint(1, width + 1, (batch, 1), generator=gen)
    lens[3] = width
    lens[4] = 1
    scores = torch.randn(batch, generator=gen)
    want, want_kl = o_adv.kl_token_level_rewards(old, ref, lens, scores, 0.05, penalty)
    for cast in (torch.int64, torch.int32):
        got, got_kl = mrl.kl_token_level_rewards(old.to(dev), ref.to(dev), lens.to(cast).to(dev), scores.to(dev), 0.05,
                                                 penalty)
        assert (got.cpu() - want).abs().max().item() < 1e-6
        assert got_kl == pytest.approx(want_kl, rel=1e-5, abs=1e-8)
    with pytest.raises(NotImplementedError):
        mrl.kl_token_level_rewards(old.to(dev), ref.to(dev), lens.to(dev), scores.to(dev), 0.05, "full")


def test_value_loss_and_critic_parity(dev):
    gen = torch.Generator().manual_seed(23)
    batch, width = 19, 53
    values = torch.randn(batch, width, generator=gen)
    vp = values + torch.randn(batch, width, generator=gen) * 0.4
    vp[0, :5] = values[0, :5]                        # ties of the two squared errors
    vp[1, :5] = values[1, :5] + 0.2                  # exactly on the edge of the clip interval
    returns = values + torch.randn(batch, width, generator=gen)
    lens = torch.randint(0, width + 1, (batch, 1), generator=gen)
    mask = o_pack.generate_mask(vp, lens).float()
    for m_o, kwargs in ((mask, dict(response_mask=mask.to(dev))), (mask, dict(response_length=lens.to(dev))),
                        (mask * 0.5, dict(response_mask=(mask * 0.5).to(dev)))):
        vo = vp.clone().requires_grad_()
        want, want_frac = o_loss.value_loss(vo, returns, values, m_o, 0.2)
        (g_o,) = torch.autograd.grad(want * 3.0, vo)
        vd = vp.to(dev).requires_grad_()
        got, out = mrl.value_loss(vd, returns.to(dev), values.to(dev), cliprange_value=0.2, loss_scale=3.0, **kwargs)
        assert got.item() == pytest.approx(3.0 * want.item(), rel=TOL_LOSS_REL)
        assert out[1].item() == pytest.approx(want.item(), rel=TOL_LOSS_REL)
        assert out[2].item() == pytest.approx(want_frac.item(), rel=1e-5, abs=1e-8)
        (g,) = torch.autograd.grad(got, vd)
        assert (g.cpu() - g_o).abs().max().item() < 1e-6
    # the loss object end to end: value head output [B, S, 1] padded, and [1, T, 1] packed
    n_seq, align = 6, 4
    plen = torch.randint(1, 5, (n_seq, 1), generator=gen, dtype=torch.int32)
    rlen = torch.randint(1, 12, (n_seq, 1), generator=gen, dtype=torch.int32)
    seq = int((plen + rlen).max())
    resp_w = int(rlen.max())
    ids = torch.ones(n_seq, seq, dtype=torch.int64)
    mask1d = o_pack.generate_mask(ids, plen + rlen)
    _, _, _, seqlens, cu = o_pack.preprocess_packed_seqs(ids, ids, mask1d, align)
    total = int(cu[-1])
    b = {"responses": torch.zeros(n_seq, resp_w, dtype=torch.int64), "prompt_length": plen, "response_length": rlen,
         "values": torch.randn(n_seq, resp_w, generator=gen), "returns": torch.randn(n_seq, resp_w, generator=gen)}
    crit = mrl.CriticLossFunc()
    crit.add_loss_meta_info({"cliprange_value": 0.3})
    cases = ((torch.randn(n_seq, seq, 1, generator=gen), {}),
             (torch.randn(1, total, 1, generator=gen), dict(use_remove_padding=True, seqlens_in_batch=seqlens,
                                                            cu_seqlens_padded=cu, seq_len=seq)))
    for out_cpu, kw in cases:
        for dyn in ({}, dict(use_dynamic_bsz=True, actual_micro_batch_size=4)):
            zo = out_cpu.clone().requires_grad_()
            want, want_stats = o_loss.critic_compute_loss(zo, b, 0.3, **kw, **dyn)
            (g_o,) = torch.autograd.grad(want, zo)
            zd = out_cpu.to(dev).requires_grad_()
            got, stats = crit.compute_loss(zd, _to_dev(b, dev), **_to_dev(kw, dev), **dyn)
            assert got.item() == pytest.approx(want.item(), rel=TOL_LOSS_REL)
            for k in want_stats:
                assert stats[k] == pytest.approx(want_stats[k], rel=TOL_LOSS_REL, abs=1e-8), k
            (g,) = torch.autograd.grad(got, zd)
            assert g.shape == out_cpu.shape and (g.cpu() - g_o).abs().max().item() < 1e-6
        vpreds = crit.compute_loss(out_cpu.to(dev), _to_dev(b, dev), forward_only=True, **_to_dev(kw, dev))
        assert torch.equal(vpreds.cpu(), o_loss.critic_compute_loss(out_cpu, b, 0.3, forward_only=True, **kw))


# --------------------------------------------------------------------------------- advantages
def test_group_advantage_parity(dev, reference_vectors):
    v = reference_vectors["group_norm_advantage"]
    adv, ret = mrl.compute_group_norm_advantage_return(
        torch.tensor(v["token_level_rewards"]), torch.tensor(v["eos_mask"]).to(dev),
        torch.tensor(v["response_length"]), v["n_sample_per_prompt"])
    assert torch.allclose(adv.cpu(), torch.tensor(v["advantages"]), atol=1e-4)
    assert torch.allclose(ret.cpu(), torch.tensor(v["returns"]), atol=1e-4)
    assert adv.data_ptr() != ret.data_ptr()
    gen = torch.Generator().manual_seed(31)
    for batch, group, width in [(128, 8, 2048), (16, 4, 256), (128, 16, 333), (6, 1, 4), (64, 64, 7), (192, 96, 9),
                                (400, 200, 5), (130, 65, 70)]:
        rewards = torch.bernoulli(torch.rand(batch // group, 1, generator=gen).repeat(1, group), generator=gen)
        rewards = rewards.reshape(batch, 1)
        rewards[:group] = 1.0                          # an all-equal group: exactly zero
        lens = torch.randint(0, width + 1, (batch,), generator=gen)
        for mask in (o_pack.generate_mask(torch.zeros(batch, width), lens),
                     o_pack.generate_mask(torch.zeros(batch, width), lens).float(),
                     o_pack.generate_mask(torch.zeros(batch, width), lens).bool()):
            want, _ = o_adv.compute_group_norm_advantage_return(rewards, mask, torch.zeros(batch, 1), group)
            got, got_ret = mrl.compute_group_norm_advantage_return(rewards.to(dev), mask.to(dev),
                                                                   torch.zeros(batch, 1), group)
            assert got.dtype == torch.float32 and got.shape == (batch, width)
            if group == 1:
                live = mask.bool()
                assert torch.isnan(got.cpu()[live]).all() and torch.isnan(want[live]).all()
                continue
            assert (got.cpu() - want).abs().max().item() < 1e-6
            assert torch.equal(got, got_ret)
            assert torch.equal(got[:group].cpu(), torch.zeros(group, width))
            # group assignment is row // G exactly: the sign pattern of each row follows its own group
            assert torch.equal((got.cpu() != 0), (want != 0))
    # gaussian rewards in fp64 and fp32, groups below, at and above the 64 lanes of the reducing wavefront
    for n, group, dtype in ((48, 6, torch.float64), (256, 64, torch.float32), (300, 100, torch.float64),
                            (63 * 3, 63, torch.float32)):
        rewards = torch.randn(n, 1, generator=gen, dtype=dtype) * 3 + 1
        mask = torch.ones(n, 3)
        want, _ = o_adv.compute_group_norm_advantage_return(rewards, mask, torch.zeros(n, 1), group)
        got, _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), mask.to(dev), torch.zeros(n, 1), group)
        assert (got.cpu() - want).abs().max().item() < 1e-6
        want_last = o_adv.get_last_reward(rewards.float(), group)
        got_last = mrl.get_last_reward(rewards.float().to(dev), group)
        assert got_last.shape == rewards.shape and (got_last.cpu() - want_last).abs().max().item() < 1e-5


def test_dynamic_sampling_keep_bit_exact(dev):
    rng = np.random.default_rng(7)
    cases = [([1, 1, 1, 1, 0, 1, 0, 0, 0.5, 0.5, 0.5, 0.5, 0, 0, 0, 1e-100], 4), ([0, 0, 0, 1e-300], 4),
             ([0.1, 0.1, 0.1], 3), ([0.1] * 4, 4), ([3.0, 3.0], 1), ([2.0, 2.0], 2), ([1, 0, 1, 1, 1], 2)]
    for n, group in [(128, 16), (128, 8), (4096, 16), (300, 7), (2048, 256), (1000, 200)]:
        p = rng.beta(0.5, 0.5, size=(n + group - 1) // group)
        vals = (rng.random(n) < np.repeat(p, group)[:n]).astype(np.float64)
        cases.append((vals.tolist(), group))
        cases.append((np.round(rng.random(n), 1).tolist(), group))     # many equal-valued groups
    for vals, group in cases:
        for dt in (torch.float64, torch.float32):
            t = torch.tensor(vals, dtype=dt)
            want = o_adv.dynamic_sampling_keep(t.numpy(), group)
            want = [i for i in want if i < len(vals)]
            got = mrl.dynamic_sampling_keep(t.to(dev), group)
            assert got == want, (vals[:8], group, dt)


# --------------------------------------------------------------------------------- policy loss
def _loss_case(gen, rows, cols):
    lp = -torch.rand(rows, cols, generator=gen) * 3
    old = lp + torch.randn(rows, cols, generator=gen) * 0.3
    ref = lp + torch.randn(rows, cols, generator=gen) * 0.3
    adv = torch.randn(rows, 1, generator=gen).repeat(1, cols)
    ent = torch.rand(rows, cols, generator=gen) * 2
    lens = torch.randint(1, cols + 1, (rows, 1), generator=gen, dtype=torch.int32)
    return lp, old, ref, adv, ent, lens


def _check_loss(got, want, g_got, g_want):
    for a, b in zip(got, want):
        a, b = float(a), float(b)
        assert abs(a - b) <= TOL_LOSS_REL * abs(b) + 1e-7, (got, want)
    for a, b in zip(g_got, g_want):
        assert (a.cpu() - b).abs().max().item() <= 1e-6 + 1e-4 * b.abs().max().item()


@pytest.mark.parametrize("kl", ["low_var_kl", "kl", "abs", "mse"])
@pytest.mark.parametrize("with_old", [True, False])
def test_grpo_policy_loss_parity(dev, kl, with_old):
    gen = torch.Generator().manual_seed(41)
    lp, old, ref, adv, ent, lens = _loss_case(gen, 16, 257)
    if not with_old:
        old = None
    ref[0, :5] = lp[0, :5] + torch.tensor([25.0, -25.0, 3.0, -3.0, 0.0])    # both k3 clamps, abs at 0
    mask = o_pack.generate_mask(lp, lens)
    lp_o, ent_o = lp.clone().requires_grad_(), ent.clone().requires_grad_()
    want = o_loss.grpo_policy_loss(old, lp_o, ref, adv, ent_o, mask, 0.2, 0.05, kl, 0.01)
    g_want = torch.autograd.grad(want[0], [lp_o, ent_o])
    ctrl = mrl.FixedKLController(0.05)
    lp_d, ent_d = lp.to(dev).requires_grad_(), ent.to(dev).requires_grad_()
    got = mrl.GRPOActorLossFunc._compute_grpo_policy_loss(
        None if old is None else old.to(dev), lp_d, ref.to(dev), adv.to(dev), ent_d, mask.to(dev), 0.2, ctrl, kl, 0.01)
    g_got = torch.autograd.grad(got[0], [lp_d, ent_d], torch.tensor(1.0, device=dev))
    _check_loss(got, want, g_got, g_want)
    # an upstream scale multiplies the gradient
    got2 = mrl.GRPOActorLossFunc._compute_grpo_policy_loss(
        None if old is None else old.to(dev), lp_d, ref.to(dev), adv.to(dev), ent_d, mask.to(dev), 0.2, ctrl, kl, 0.01)
    (g2,) = torch.autograd.grad(got2[0] * 0.125, [lp_d])
    assert torch.allclose(g2, g_got[0] * 0.125, atol=1e-9)


def test_policy_loss_ties_clip_edges_and_nan_outside_mask(dev):
    # ratio exactly on the clip bounds, zero advantages (ties), NaN outside the mask
    lo, hi = float(np.float32(1.0 - 0.2)), float(np.float32(1.0 + 0.2))
    old = torch.zeros(1, 8)
    lp = torch.tensor([[math.log(lo), math.log(hi), 0.0, 0.5, -0.5, 0.1, float("nan"), 0.3]])
    adv = torch.tensor([[1.0, -1.0, 0.0, 0.0, 0.0, -2.0, 1.0, float("nan")]])
    mask = torch.tensor([[1, 1, 1, 1, 1, 1, 0, 0]])
    ent = torch.zeros(1, 8)
    lp_o = lp.clone().requires_grad_()
    want = o_loss.grpo_policy_loss(old, lp_o, lp.detach().clone(), adv, ent, mask, 0.2, 0.0, "low_var_kl", 0.0)
    (g_want,) = torch.autograd.grad(want[0], lp_o)
    lp_d = lp.to(dev).requires_grad_()
    got = mrl.GRPOActorLossFunc._compute_grpo_policy_loss(old.to(dev), lp_d, lp.to(dev), adv.to(dev), ent.to(dev),
                                                           mask.to(dev), 0.2, mrl.FixedKLController(0.0),
                                                           "low_var_kl", 0.0)
    (g_got,) = torch.autograd.grad(got[0], lp_d)
    assert not math.isnan(float(got[0]))
    _check_loss(got, want, [g_got[:, :6]], [g_want[:, :6]])
    assert torch.equal(g_got[:, 6:].cpu(), torch.zeros(1, 2))


@pytest.mark.parametrize("token_level", [True, False])
def test_dapo_policy_loss_parity(dev, token_level, reference_vectors):
    v = reference_vectors["dapo_policy_loss_inputs"]
    t = {k: torch.tensor(v[k], dtype=torch.float32) for k in ("old_log_prob", "log_prob", "entropy", "advantages",
                                                              "eos_mask")}
    for old in (t["old_log_prob"], None):
        want = o_loss.dapo_policy_loss(old, t["log_prob"], t["entropy"], v["entropy_coeff"], t["advantages"],
                                       t["eos_mask"], v["clip_ratio_low"], v["clip_ratio_high"], token_level)
        got = mrl.DAPOActorLossFunc._compute_dapo_policy_loss(
            None if old is None else old.to(dev), t["log_prob"].to(dev), t["entropy"].to(dev), v["entropy_coeff"],
            t["advantages"].to(dev), t["eos_mask"].to(dev), v["clip_ratio_low"], v["clip_ratio_high"], token_level)
        assert len(got) == 5 and all(isinstance(x, torch.Tensor) for x in got)
        _check_loss(got, want, [], [])
    gen = torch.Generator().manual_seed(43)
    lp, old, _, adv, ent, lens = _loss_case(gen, 24, 500)
    mask = o_pack.generate_mask(lp, lens).float()
    lp_o, ent_o = lp.clone().requires_grad_(), ent.clone().requires_grad_()
    want = o_loss.dapo_policy_loss(old, lp_o, ent_o, 0.003, adv, mask, 0.2, 0.28, token_level)
    g_want = torch.autograd.grad(want[0], [lp_o, ent_o])
    lp_d, ent_d = lp.to(dev).requires_grad_(), ent.to(dev).requires_grad_()
    got = mrl.DAPOActorLossFunc._compute_dapo_policy_loss(old.to(dev), lp_d, ent_d, 0.003, adv.to(dev), mask.to(dev),
                                                           0.2, 0.28, token_level)
    g_got = torch.autograd.grad(got[0], [lp_d, ent_d])
    _check_loss(got, want, g_got, g_want)
    assert float(got[3]) == 0.0
    if not token_level:
        assert float(got[1]) == 0.0                    # the reference's overwritten-operand clip fraction
        mask[3] = 0                                    # an all-masked row: NaN, as in the reference
        got = mrl.DAPOActorLossFunc._compute_dapo_policy_loss(old.to(dev), lp.to(dev), ent.to(dev), 0.0, adv.to(dev),
                                                               mask.to(dev), 0.2, 0.28, False)
        assert math.isnan(float(got[0]))


# --------------------------------------------------------------------------------- end to end
def _make_batch(gen, n_prompts, group, r_lo, r_hi, vocab, dtype, scale, align, prompt_hi=2):
    """Synthetic GRPO micro-batch in the layout the training engine hands to the loss."""
    batch = n_prompts * group
    rlen = torch.randint(r_lo, r_hi + 1, (batch, 1), generator=gen, dtype=torch.int32)
    plen = torch.randint(1, prompt_hi + 1, (batch, 1), generator=gen, dtype=torch.int32)
    width = int((plen + rlen).max())
    resp_w = int(rlen.max())
    ids = torch.randint(0, vocab, (batch, width), generator=gen)
    mask1d = o_pack.generate_mask(ids, plen + rlen)
    ids = ids * mask1d
    labels = torch.cat([ids[:, 1:], torch.zeros(batch, 1, dtype=ids.dtype)], 1)
    p_ids, _, p_lab, seqlens, cu = o_pack.preprocess_packed_seqs(ids, labels, mask1d, align)
    total = p_ids.shape[1]
    logits = (torch.randn(1, total, vocab, generator=gen) * scale).to(dtype)
    p = torch.rand(n_prompts, 1, generator=gen).repeat(1, group).reshape(batch, 1)
    rewards = torch.bernoulli(p, generator=gen)
    rmask = o_pack.generate_mask(torch.zeros(batch, resp_w), rlen)
    adv, _ = o_adv.compute_group_norm_advantage_return(rewards, rmask, rlen, group)
    b = {"labels": p_lab, "responses": torch.zeros(batch, resp_w, dtype=torch.int32), "response_length": rlen,
         "prompt_length": plen, "advantages": adv}
    kw = dict(use_remove_padding=True, seqlens_in_batch=seqlens, cu_seqlens_padded=cu, seq_len=width)
    # behaviour / reference policy log-probs: current + N(0, 0.05), from the oracle, detached
    lp0 = o_loss.logprob_computer(logits.float(), b, True, **kw)[0]
    b["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    b["ref_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    return logits, b, kw, rewards, (ids, labels, mask1d)


def _to_dev(d, dev):
    return {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in d.items()}


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("entropy_coeff", [0.0, 0.001])
def test_grpo_compute_loss_config0_packed(dev, entropy_coeff, fused):
    """configs[0]: 4 prompts x G=4, R in [64,256], V=32000 fp32 logits ~N(0,2), eps 0.2, k3 KL 0.001."""
    gen = torch.Generator().manual_seed(0)
    logits, b, kw, rewards, _ = _make_batch(gen, 4, 4, 64, 256, 32000, torch.float32, 2.0, 1, prompt_hi=1)
    meta = dict(clip_ratio=0.2, kl_coef=0.001, kl_penalty="low_var_kl", entropy_coeff=entropy_coeff)
    zo = logits.clone().requires_grad_()
    want_loss, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want_loss, zo)

    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.001), "kl_penalty": "low_var_kl",
                          "entropy_coeff": entropy_coeff})
    zd = logits.to(dev).requires_grad_()
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    kwd["fused"] = fused        # one-sweep eager gradient, or the split forward / backward kernels
    # advantages computed on the device from the rewards agree with the oracle's
    rmask = mrl.generate_mask(bd["responses"], bd["response_length"])
    adv_d, _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), rmask, bd["response_length"], 4)
    assert (adv_d.cpu() - b["advantages"]).abs().max().item() < 1e-6
    lp = f.compute_loss(zd, bd, forward_only=True, **kwd)
    lp_o = o_loss.grpo_compute_loss(logits, b, meta, forward_only=True, **kw)
    assert lp.shape == lp_o.shape and (lp.cpu() - lp_o).abs().max().item() < TOL_LOGP
    loss, stats = f.compute_loss(zd, bd, **kwd)
    assert loss.dim() == 0 and set(stats) == set(want_stats)
    assert all(isinstance(x, float) for x in stats.values())
    assert abs(loss.item() - want_loss.item()) <= TOL_LOSS_REL * abs(want_loss.item()) + 1e-7
    for k in want_stats:
        assert abs(stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    (dz,) = torch.autograd.grad(loss, zd)
    assert (dz.cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    scale = dz_o.abs().max().item()
    assert (dz.cpu() - dz_o).abs().max().item() < 1e-3 * scale + 1e-9      # relative, since dlogits are tiny
    # Megatron scales the loss before backward: the gradient follows
    (dz2,) = torch.autograd.grad(f.compute_loss(zd, bd, **kwd)[0] * 64.0, zd)
    assert torch.allclose(dz2, dz * 64.0, rtol=1e-5, atol=1e-12)
    # dynamic batch size rescales the loss only
    loss3, stats3 = f.compute_loss(zd, bd, use_dynamic_bsz=True, actual_micro_batch_size=4.0, **kwd)
    assert loss3.item() == pytest.approx(loss.item() * 4.0, rel=1e-6) and stats3 == stats
    ref = mrl.LossFuncFactory.get_instance("ray_grpo", "reference")
    assert torch.equal(ref.compute_loss(zd, bd, forward_only=True, **kwd), lp)
    assert ref.compute_loss(zd, bd, forward_only=False, **kwd) is None
    with pytest.raises(ValueError, match="The responses is None"):
        f.compute_loss(zd, {k: v for k, v in bd.items() if k != "responses"},
                       **{k: v for k, v in kwd.items() if k != "use_remove_padding"})


@pytest.mark.parametrize("fused", [True, False])
def test_padded_vs_packed_and_dapo_bf16(dev, fused):
    """configs[2]/[4] in small: the same responses as a padded [B,S] batch and packed with
    alignment 8, bf16 logits, an empty-response group, DAPO clip-higher with sequence mean."""
    gen = torch.Generator().manual_seed(2)
    logits, b, kw, rewards, (ids, labels, mask1d) = _make_batch(gen, 3, 4, 5, 40, 4096, torch.bfloat16, 3.0, 8)
    b["response_length"][4:8] = 0            # note: lengths only shrink the loss mask here
    meta = dict(entropy_coeff=0.002, token_level_loss=True, clip_higher_enable=True, clip_ratio_low=0.2,
                clip_ratio_high=0.28)
    batch, width = ids.shape
    seqlens, cu = kw["seqlens_in_batch"], kw["cu_seqlens_padded"]
    padded = torch.zeros(batch, width, 4096, dtype=torch.bfloat16)
    for i in range(batch):
        padded[i, :seqlens[i]] = logits[0, cu[i]:cu[i] + seqlens[i]]
    f = mrl.LossFuncFactory.get_instance("ray_dapo", "actor")
    f.add_loss_meta_info({"entropy_coeff": 0.002, "token_level_loss": True, "clip_higher_enable": True,
                          "clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "clip_ratio": 0.2})
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    kwd["fused"] = fused
    zo = logits.float().requires_grad_()
    want_loss, want_stats = o_loss.dapo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want_loss, zo)
    zd = logits.to(dev).requires_grad_()
    loss, stats = f.compute_loss(zd, bd, **kwd)
    assert abs(loss.item() - want_loss.item()) <= TOL_LOSS_REL * abs(want_loss.item()) + 1e-7
    for k in want_stats:
        assert abs(stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    (dz,) = torch.autograd.grad(loss, zd)
    assert dz.dtype == torch.bfloat16
    assert (dz.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    # padded layout through the same loss object: same loss, same statistics
    bp = dict(bd, labels=labels.to(dev))
    zp = padded.to(dev).requires_grad_()
    loss_p, stats_p = f.compute_loss(zp, bp, fused=fused)
    assert loss_p.item() == pytest.approx(loss.item(), rel=1e-6)
    for k in stats:
        assert stats_p[k] == pytest.approx(stats[k], rel=1e-6, abs=1e-9)
    (dzp,) = torch.autograd.grad(loss_p, zp)
    for i in range(batch):
        assert torch.equal(dzp[i, :seqlens[i]].cpu(), dz[0, cu[i]:cu[i] + seqlens[i]].cpu())
    # sequence-mean mode and a response mask handed in by the caller
    f.add_loss_meta_info({"token_level_loss": False})
    meta["token_level_loss"] = False
    b2 = dict(b, response_length=torch.clamp(b["response_length"], min=1))
    rm = o_pack.generate_mask(b["responses"], b2["response_length"]).float()
    rm[:, ::3] = 0
    rm[:, 0] = 1
    b2["response_mask"] = rm
    zo2 = logits.float().requires_grad_()
    want_loss, want_stats = o_loss.dapo_compute_loss(zo2, b2, meta, **kw)
    (dz_o2,) = torch.autograd.grad(want_loss, zo2)
    loss, stats = f.compute_loss(zd, _to_dev(b2, dev), **kwd)
    assert abs(loss.item() - want_loss.item()) <= TOL_LOSS_REL * abs(want_loss.item()) + 1e-7
    assert stats["actor/pg_clipfrac"] == 0.0 and stats["actor/kl_loss"] == 0.0
    (dz2,) = torch.autograd.grad(loss, zd)
    assert (dz2.float().cpu() - dz_o2).abs().max().item() < TOL_DLOGITS
    assert (dz2.float().cpu() - dz_o2).abs().max().item() < 1e-2 * dz_o2.abs().max().item()


@pytest.mark.parametrize("fused", [True, False])
def test_padded_vs_packed_full_vocab_grpo(dev, fused):
    """configs[2] at the configs[1] row shape (V=152064, bf16), batch scaled down: GRPO loss on the
    padded [B,S,V] layout and on the packed one, with a group of empty responses and a group whose
    rewards are all equal (std 0: the eps keeps its advantages at exactly zero, so only the KL
    term drives those rows)."""
    gen = torch.Generator().manual_seed(22)
    group, vocab = 4, 152064
    logits, b, kw, rewards, (ids, labels, mask1d) = _make_batch(gen, 3, group, 6, 30, vocab, torch.bfloat16, 3.0, 1)
    rewards[:group] = 1.0                                   # all-equal group
    rewards[2 * group:, 0] = torch.tensor([1.0, 0.0, 0.0, 1.0])
    b["response_length"][group:2 * group] = 0               # group of empty responses
    rmask = o_pack.generate_mask(b["responses"], b["response_length"])
    b["advantages"], _ = o_adv.compute_group_norm_advantage_return(rewards, rmask, b["response_length"], group)
    assert torch.equal(b["advantages"][:group], torch.zeros_like(b["advantages"][:group]))
    assert b["advantages"][2 * group:].abs().max() > 0.5
    adv_d, _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), rmask.to(dev), b["response_length"].to(dev),
                                                       group)
    assert (adv_d.cpu() - b["advantages"]).abs().max().item() < TOL_LOGP
    assert torch.equal(adv_d[:2 * group].cpu(), torch.zeros_like(b["advantages"][:2 * group]))
    meta = dict(clip_ratio=0.2, kl_coef=0.001, kl_penalty="low_var_kl", entropy_coeff=0.001)
    zo = logits.float().requires_grad_()
    want_loss, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want_loss, zo)
    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.001), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.001})
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    zd = logits.to(dev).requires_grad_()
    loss, stats = f.compute_loss(zd, bd, fused=fused, **kwd)
    assert abs(loss.item() - want_loss.item()) <= TOL_LOSS_REL * abs(want_loss.item()) + 1e-7
    for k in want_stats:
        assert abs(stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    (dz,) = torch.autograd.grad(loss, zd)
    assert (dz.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    # rows of the empty-response group carry no gradient at all
    seqlens, cu = kw["seqlens_in_batch"], kw["cu_seqlens_padded"]
    for i in range(group, 2 * group):
        assert not dz[0, cu[i]:cu[i] + seqlens[i]].any().item()
    # the same responses in the padded layout: same loss and statistics, bit-identical gradient rows,
    # zero gradient on the padding rows
    batch, width = ids.shape
    padded = torch.randn(batch, width, vocab, generator=gen).to(torch.bfloat16)     # padding rows hold noise
    for i in range(batch):
        padded[i, :seqlens[i]] = logits[0, cu[i]:cu[i] + seqlens[i]]
    zp = padded.to(dev).requires_grad_()
    loss_p, stats_p = f.compute_loss(zp, dict(bd, labels=labels.to(dev)), fused=fused)
    assert loss_p.item() == pytest.approx(loss.item(), rel=1e-6)
    for k in stats:
        assert stats_p[k] == pytest.approx(stats[k], rel=1e-6, abs=1e-9)
    (dzp,) = torch.autograd.grad(loss_p, zp)
    for i in range(batch):
        assert torch.equal(dzp[i, :seqlens[i]], dz[0, cu[i]:cu[i] + seqlens[i]])
        assert not dzp[i, seqlens[i]:].any().item()


@pytest.mark.parametrize("fused", [True, False])
def test_ppo_actor_loss_parity(dev, fused):
    """PPO actor (the GRPO surrogate without KL, four statistics), end to end and as a stand-alone op."""
    gen = torch.Generator().manual_seed(17)
    logits, b, kw, _, _ = _make_batch(gen, 2, 3, 4, 20, 4096, torch.bfloat16, 3.0, 1)
    meta = dict(clip_ratio=0.25, entropy_coeff=0.004)
    zo = logits.float().requires_grad_()
    want, want_stats = o_loss.ppo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want, zo)
    f = mrl.LossFuncFactory.get_instance("ray_ppo", "actor")
    assert isinstance(f, mrl.PPOActorLossFunc)
    f.add_loss_meta_info({"clip_ratio": 0.25, "entropy_coeff": 0.004, "kl_ctrl": mrl.FixedKLController(0.1)})
    zd = logits.to(dev).requires_grad_()
    got, got_stats = f.compute_loss(zd, _to_dev(b, dev), fused=fused, **_to_dev(kw, dev))
    assert set(got_stats) == set(want_stats) == {"actor/pg_loss", "actor/pg_clipfrac", "actor/ppo_kl", "actor/entropy"}
    assert abs(got.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    for k in want_stats:
        assert abs(got_stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    (dz,) = torch.autograd.grad(got, zd)
    assert (dz.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    lp, old, _, adv, ent, lens = _loss_case(gen, 8, 33)
    mask = o_pack.generate_mask(lp, lens)
    want4 = o_loss.ppo_policy_loss(old, lp, adv, mask, 0.2, ent, 0.01)
    got4 = mrl.PPOActorLossFunc._compute_ppo_policy_loss(old.to(dev), lp.to(dev), adv.to(dev), mask.to(dev), 0.2,
                                                         ent.to(dev), 0.01)
    assert len(got4) == 4
    _check_loss(got4, want4, [], [])


def test_fused_sweep_specifics(dev):
    """The one-sweep path: agreement with the split kernels, an upstream scale that differs from
    the expected one (rescale kernel), in-place gradients, tokens whose mask reaches past the
    logits window, and the automatic fall-back for a vocabulary the registers cannot hold."""
    gen = torch.Generator().manual_seed(7)
    logits, b, kw, _, _ = _make_batch(gen, 2, 4, 6, 30, 8192, torch.bfloat16, 3.0, 2, prompt_hi=3)
    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.003})
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    assert mrl.fused_supported(logits.to(dev))
    zd = logits.to(dev).requires_grad_()
    loss_s, stats_s = f.compute_loss(zd, bd, fused=False, **kwd)
    (dz_s,) = torch.autograd.grad(loss_s, zd)
    loss_f, stats_f = f.compute_loss(zd, bd, fused=True, **kwd)
    (dz_f,) = torch.autograd.grad(loss_f, zd)
    # the two paths sum the row in a different order, and the surrogate is a cancelling sum of +-A*r
    assert loss_f.item() == pytest.approx(loss_s.item(), rel=5e-5)
    for k in stats_s:
        assert stats_f[k] == pytest.approx(stats_s[k], rel=5e-5, abs=1e-8)
    assert (dz_f.float() - dz_s.float()).abs().max().item() <= 2 ** -8 * dz_s.float().abs().max().item()
    # upstream 1/16 while 1 was expected: the stored gradient is rescaled; expected 1/16: no rescale needed
    (dz_16,) = torch.autograd.grad(f.compute_loss(zd, bd, fused=True, **kwd)[0] / 16.0, zd)
    assert torch.equal(dz_16.float() * 16.0, dz_f.float())
    (dz_16b,) = torch.autograd.grad(f.compute_loss(zd, bd, fused=True, expected_grad_scale=1 / 16.0, **kwd)[0] / 16.0, zd)
    assert torch.equal(dz_16b, dz_16)
    # in place: the gradient lands in the logits buffer
    z_in = logits.to(dev).requires_grad_()
    loss_i, _ = f.compute_loss(z_in, bd, fused=True, grad_inplace=True, **kwd)
    (dz_i,) = torch.autograd.grad(loss_i, z_in)
    assert dz_i.data_ptr() == z_in.data_ptr() and torch.equal(dz_i, dz_f)
    # a mask that reaches past the window (response_length larger than what the packed rows hold)
    b2 = dict(b, response_length=b["response_length"] + 2)
    width = b["responses"].shape[1]
    b2["response_length"] = torch.clamp(b2["response_length"], max=width)
    want, want_stats = o_loss.grpo_compute_loss(logits.float(), b2, dict(clip_ratio=0.2, kl_coef=0.01,
                                                kl_penalty="low_var_kl", entropy_coeff=0.003), **kw)
    got, got_stats = f.compute_loss(zd, _to_dev(b2, dev), fused=True, **kwd)
    assert abs(got.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    for k in want_stats:
        assert abs(got_stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    # no old_log_prob: ratio 1
    b3 = {k: v for k, v in b.items() if k != "old_log_prob"}
    zo = logits.float().requires_grad_()
    want, _ = o_loss.grpo_compute_loss(zo, b3, dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl",
                                                    entropy_coeff=0.003), **kw)
    (dz_o,) = torch.autograd.grad(want, zo)
    got, _ = f.compute_loss(zd, _to_dev(b3, dev), fused=True, **kwd)
    (dz_g,) = torch.autograd.grad(got, zd)
    assert abs(got.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    assert (dz_g.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    # a vocabulary that is not a multiple of the vector width falls back to the split kernels
    odd = torch.randn(1, logits.shape[1], 1003, generator=gen).to(torch.bfloat16).to(dev).requires_grad_()
    assert not mrl.fused_supported(odd)
    bd_odd = dict(bd, labels=bd["labels"] % 1003)
    loss_o, _ = f.compute_loss(odd, bd_odd, fused=True, **kwd)
    (dz_odd,) = torch.autograd.grad(loss_o, odd)
    assert dz_odd.shape == odd.shape and torch.isfinite(loss_o).item()
    assert _lib.load().mrl_fused_max_vocab(_lib.BF16) == 2 * 19 * 1024 * 8
    assert _lib.load().mrl_fused_max_vocab(_lib.F32) == 2 * 19 * 1024 * 4


@pytest.mark.parametrize("dtype,vocab", [(torch.bfloat16, 152064), (torch.bfloat16, 129280), (torch.float32, 32000),
                                         (torch.float16, 65536), (torch.float32, 77824), (torch.bfloat16, 64),
                                         (torch.float32, 152064), (torch.bfloat16, 262144), (torch.float32, 77828),
                                         (torch.float16, 311296), (torch.float32, 100004)])
def test_fused_sweep_vocab_sizes(dev, dtype, vocab):
    """Every register-tile size of the fused kernel (4, 8, 12, 16, 19 vectors per thread), and rows
    that two workgroups hold (fp32 logits of the configs[1] vocabulary, a 256 k vocabulary in bf16,
    the first and the last width of that kind, an odd number of vectors)."""
    gen = torch.Generator().manual_seed(vocab)
    logits, b, kw, _, _ = _make_batch(gen, 1, 4, 3, 9, vocab, dtype, 3.0, 1, prompt_hi=2)
    meta = dict(clip_ratio=0.2, kl_coef=0.02, kl_penalty="low_var_kl", entropy_coeff=0.002)
    zo = logits.float().requires_grad_()
    want, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want, zo)
    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.02), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.002})
    zd = logits.to(dev).requires_grad_()
    assert mrl.fused_supported(zd)
    got, got_stats = f.compute_loss(zd, _to_dev(b, dev), fused=True, **_to_dev(kw, dev))
    (dz,) = torch.autograd.grad(got, zd)
    assert abs(got.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    for k in want_stats:
        assert abs(got_stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    assert (dz.float().cpu() - dz_o).abs().max().item() < TOL_DLOGITS
    assert (dz.float().cpu() - dz_o).abs().max().item() <= 2 ** -8 * dz_o.abs().max().item() + 1e-9
    # the gradient written over the logits, and - for rows that two workgroups hold - without ever waiting
    # for the other half's record (every workgroup reads the other half itself): the same bits
    lib = _lib.load()
    for limit in (-1, 0):
        lib.mrl_set_wide_spin_limit(limit)
        try:
            z2 = logits.to(dev).requires_grad_()
            z_in = z2 * 1.0
            got2, _ = f.compute_loss(z_in, _to_dev(b, dev), fused=True, grad_inplace=True, **_to_dev(kw, dev))
            (dz2,) = torch.autograd.grad(got2, z2)
        finally:
            lib.mrl_set_wide_spin_limit(-1)
        assert got2.item() == got.item() and torch.equal(dz2, dz), limit


@pytest.mark.parametrize("dtype,vocab", [(torch.float32, 152064), (torch.bfloat16, 262144)])
def test_fused_sweep_wide_rows(dev, dtype, vocab):
    """Rows that two workgroups hold: more half rows than workgroups (tickets are recycled, partners
    change), fused against the split kernels and an fp32 torch chain on the device; twice on one
    stream and on two streams at once with a workspace each, then captured in a graph and replayed
    with an eager sweep next to it - bit-identical to a lone call every time (both halves of a row
    merge the two records in the same order)."""
    rows = 700
    gen = torch.Generator(device=dev).manual_seed(vocab)
    cases = []
    for c in range(2):
        z = (torch.randn(rows, vocab, generator=gen, device=dev) * 3).to(dtype)
        y = torch.randint(0, vocab, (rows,), generator=gen, device=dev)
        y[5], y[6] = -1, vocab
        ops = torch.zeros(rows, 8, device=dev)
        ops[:, 0] = -torch.rand(rows, generator=gen, device=dev) * 8
        ops[:, 1] = -torch.rand(rows, generator=gen, device=dev) * 8
        ops[:, 2] = torch.randn(rows, generator=gen, device=dev)
        ops[:, 3] = (torch.rand(rows, generator=gen, device=dev) > 0.2).float()
        ops[:, 4] = 1.0 / rows
        ops[:, 5] = 1.0 / rows
        cases.append((z, y, ops))
    lib = _lib.load()
    ws_bytes = lib.mrl_fused_workspace_bytes(_lib.dtype_code(cases[0][0]), rows, vocab)
    assert ws_bytes == 16 + rows * 32

    def outputs():
        return (torch.empty(rows, vocab, dtype=dtype, device=dev), torch.empty(rows, device=dev),
                torch.empty(rows, 8, device=dev))

    def sweep(case, out, ws, stream):
        z, y, ops = case
        dz, ent, terms = out
        _lib.call("mrl_fused_logprob_loss", z.data_ptr(), _lib.dtype_code(z), rows, vocab, vocab, y.data_ptr(),
                  _lib.I64, 1.0, ops.data_ptr(), 1, 0.8, 1.2, 3, 0.01, 0.002, 1.0, None, dz.data_ptr(), vocab, None,
                  ent.data_ptr(), terms.data_ptr(), ws.data_ptr(), ws_bytes, 0, stream)

    spaces = [torch.full((ws_bytes,), 0xCD, dtype=torch.uint8, device=dev) for _ in range(3)]
    want = []
    for case in cases:
        out = outputs()
        sweep(case, out, spaces[0], _lib.stream(dev))
        torch.cuda.synchronize()
        want.append(out)
        z, y, ops = case
        dz, ent, terms = out
        # the split kernels on the same rows (independent code): log-prob, entropy and the gradient
        lp_s, ent_s, lse_s = mrl.vocab_logprob_entropy(z, y)
        live = ops[:, 3] != 0
        assert (ent[live] - ent_s[live]).abs().max().item() < 2e-5
        assert not dz[~live].any().item() and dz[live].float().abs().amax(-1).min().item() > 0
        # an fp32 torch chain on a slice of the rows
        pick = torch.arange(0, rows, 23, device=dev)
        zr = z[pick].float().requires_grad_()
        logsm = torch.log_softmax(zr, -1)
        yp = y[pick]
        y_ok = (yp >= 0) & (yp < vocab)
        lp_ref = torch.where(y_ok, logsm.gather(-1, yp.clamp(0, vocab - 1)[:, None])[:, 0],
                             zr.max(-1).values.detach() - torch.logsumexp(zr, -1))
        p = logsm.exp()
        h_ref = -(p * logsm).sum(-1)
        old, ref, adv, m, wpg, invtok = [ops[pick, k] for k in range(6)]
        ratio = torch.exp(lp_ref - old)
        pg = torch.maximum(-adv * ratio, -adv * ratio.clamp(0.8, 1.2))
        kl = 0.5 * (lp_ref - ref) ** 2
        loss = (pg * m * wpg).sum() + 0.01 * (kl * m * invtok).sum() - 0.002 * (h_ref * m * invtok).sum()
        (g_ref,) = torch.autograd.grad(loss, zr)
        scale = g_ref.abs().max().item()
        rel = 2 ** -7 if dtype != torch.float32 else 2e-5
        assert (dz[pick].float() - g_ref).abs().max().item() <= rel * scale + 1e-9
        assert (lp_s[pick][m != 0] - lp_ref.detach()[m != 0]).abs().max().item() < 2e-4
    # again on the same stream, and two sweeps at once on two streams
    streams = [torch.cuda.Stream(device=dev) for _ in cases]
    outs = [outputs() for _ in cases]
    torch.cuda.synchronize()
    for _ in range(3):
        for case, out, s, ws in zip(cases, outs, streams, spaces):
            sweep(case, out, ws, s.cuda_stream)
    torch.cuda.synchronize()
    for got, ref in zip(outs, want):
        for a, b in zip(got, ref):
            assert torch.equal(a, b)
    # in place (the gradients overwrite the logits while other workgroups still exchange statistics), and
    # with a wait bound of zero polls: every workgroup then reads the other half of its row itself and
    # looks for the record only afterwards - out of place and in place, the same bits as above
    for limit, inplace in ((-1, True), (0, False), (0, True)):
        lib.mrl_set_wide_spin_limit(limit)
        try:
            for case, ref in zip(cases, want):
                z, y, ops = case
                dz, ent, terms = outputs()
                if inplace:
                    dz.copy_(z)
                    sweep((dz, y, ops), (dz, ent, terms), spaces[0], _lib.stream(dev))
                else:
                    sweep(case, (dz, ent, terms), spaces[0], _lib.stream(dev))
                torch.cuda.synchronize()
                for a, b in zip((dz, ent, terms), ref):
                    assert torch.equal(a, b), (limit, inplace)
        finally:
            lib.mrl_set_wide_spin_limit(-1)
    # captured once, replayed next to an eager sweep
    g_out = outputs()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sweep(cases[0], g_out, spaces[2], _lib.stream(dev))
    side = torch.cuda.Stream(device=dev)
    for i in range(3):
        for t in g_out:
            t.zero_()
        other = outputs()
        torch.cuda.synchronize()
        sweep(cases[1], other, spaces[1], side.cuda_stream)
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(g_out, want[0]):
            assert torch.equal(a, b), i
        for a, b in zip(other, want[1]):
            assert torch.equal(a, b), i


@pytest.mark.parametrize("dtype,vocab", [(torch.bfloat16, 8200), (torch.float32, 4100), (torch.float16, 40960)])
def test_persistent_row_sweeps(dev, dtype, vocab):
    """More rows than twice the CU count, rows from 16 KiB on: the streaming backward of the split
    path (one vector per thread, workgroups of 256 vectors), with rows that are skipped (no gradient)
    next to each other, at the ends and 256 rows apart, labels outside the vocabulary and in the last
    chunk of a row, a row length that does not fill the last workgroup."""
    gen = torch.Generator().manual_seed(vocab)
    rows = 700
    z = _logits(gen, rows, vocab, dtype)
    y = torch.randint(0, vocab, (rows,), generator=gen)
    y[5], y[300], y[699] = -100, vocab + 5, vocab
    g_lp = torch.randn(rows, generator=gen) * 0.1
    g_h = torch.randn(rows, generator=gen) * 0.01
    dead = [0, 1, 2, 255, 256, 257, 258, 511, 512, 513, 698, 699]
    g_lp[dead] = 0.0
    g_h[dead] = 0.0
    g_h[40:60] = 0.0                                     # log-prob gradient only
    g_lp[70:90] = 0.0                                    # entropy gradient only
    zo = z.float().requires_grad_()
    lp_o = o_vocab.compute_log_probs(zo, y)
    h_o = o_vocab.vocab_parallel_entropy(zo)
    (dz_o,) = torch.autograd.grad((lp_o * g_lp).sum() + (h_o * g_h).sum(), zo)
    zd = z.to(dev).requires_grad_()
    lp, h, lse = mrl.vocab_logprob_entropy(zd, y.to(dev))
    assert (lp.cpu() - lp_o.detach()).abs().max().item() < 1e-4
    (dz,) = torch.autograd.grad([lp, h], zd, [g_lp.to(dev), g_h.to(dev)])
    tol = 1e-5 if dtype == torch.float32 else TOL_DLOGITS
    assert (dz.float().cpu() - dz_o).abs().max().item() < tol
    assert not dz[dead].any().item()
    assert torch.equal(zd.detach().cpu(), z)
    # log-prob gradient alone (the kernel variant without the entropy term), in place over the logits
    (dz_lp_o,) = torch.autograd.grad((o_vocab.compute_log_probs(zo, y) * g_lp).sum(), zo)
    zin = z.to(dev).clone()
    gd, yd = g_lp.to(dev), y.to(dev)
    _lib.call("mrl_vocab_logprob_bwd", zin.data_ptr(), _lib.dtype_code(zin), rows, vocab, vocab, yd.data_ptr(), _lib.I64,
              1.0, lse.data_ptr(), None, gd.data_ptr(), None, zin.data_ptr(), _lib.dtype_code(zin), vocab,
              _lib.stream(dev))
    torch.cuda.synchronize()
    assert (zin.float().cpu() - dz_lp_o).abs().max().item() < tol


@pytest.mark.parametrize("rows", [5, 600])
def test_backward_fp32_full_vocab(dev, rows):
    """fp32 rows of 152064 entries (608 KiB, more than a workgroup's registers hold) through the split
    backward against the closed form; labels on both sides of a workgroup's chunk boundary (256 vectors
    of 4 entries), first, last and outside the vocabulary."""
    torch.manual_seed(rows)
    vocab = 152064
    z = (torch.randn(rows, vocab, device=dev) * 3)
    y = torch.randint(0, vocab, (rows,), device=dev)
    half = 74 * 1024
    y[0], y[1], y[2], y[3], y[4] = half - 1, half, 0, vocab - 1, -100
    g_lp = torch.randn(rows, device=dev) * 0.1
    g_h = torch.randn(rows, device=dev) * 0.01
    g_lp[2], g_h[2] = 0.0, 0.0
    zr = z.clone().requires_grad_()
    lp, h, lse = mrl.vocab_logprob_entropy(zr, y)
    (dz,) = torch.autograd.grad([lp, h], zr, [g_lp, g_h])
    ref = torch.log_softmax(z, -1)
    p = ref.exp()
    y_ok = (y >= 0) & (y < vocab)
    onehot = torch.zeros_like(z)
    onehot[y_ok, y[y_ok]] = 1.0
    closed = g_lp[:, None] * (onehot - p) - g_h[:, None] * p * (z - (p * z).sum(-1, keepdim=True))
    assert (dz - closed).abs().max().item() < 1e-5
    assert not dz[2].any().item()
    assert torch.equal(zr.detach(), z)


def test_fused_sweep_persistent_with_skipped_rows(dev):
    """The fused sweep on more than 2 x CU-count rows: prompt rows, alignment padding and sequences
    without a response are rows it must not read but must zero."""
    gen = torch.Generator().manual_seed(21)
    logits, b, kw, _, _ = _make_batch(gen, 6, 4, 20, 40, 8200, torch.bfloat16, 3.0, 4, prompt_hi=4)
    assert logits.shape[1] > 600
    b["response_length"][8:12] = 0
    b["old_log_prob"][8:12] = 0
    b["ref_log_prob"][8:12] = 0
    meta = dict(clip_ratio=0.2, kl_coef=0.02, kl_penalty="low_var_kl", entropy_coeff=0.002)
    zo = logits.float().requires_grad_()
    want, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want, zo)
    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.02), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.002})
    for coeff in (0.002, 0.0):
        if coeff == 0.0:
            meta["entropy_coeff"] = 0.0
            f.add_loss_meta_info({"entropy_coeff": 0.0})
            zo = logits.float().requires_grad_()
            want, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
            (dz_o,) = torch.autograd.grad(want, zo)
        zd = logits.to(dev).requires_grad_()
        got, got_stats = f.compute_loss(zd, _to_dev(b, dev), fused=True, **_to_dev(kw, dev))
        (dz,) = torch.autograd.grad(got, zd)
        assert abs(got.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
        for k in want_stats:
            assert abs(got_stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
        assert (dz.float().cpu() - dz_o).abs().max().item() <= 2 ** -8 * dz_o.abs().max().item() + 1e-9
        assert torch.equal(dz.float().cpu() != 0, dz_o != 0) or \
            ((dz.float().cpu() != 0) <= (dz_o != 0)).all().item()      # nothing outside the response rows


def test_fused_sweep_persistent_full_vocab(dev):
    """The persistent fused sweep at the Qwen2.5 vocabulary (19 vectors per thread, the last one partly
    past the end of the row) on more than 2 x CU-count rows, against the oracle end to end."""
    gen = torch.Generator().manual_seed(33)
    logits, b, kw, _, _ = _make_batch(gen, 2, 4, 120, 150, 152064, torch.bfloat16, 3.0, 1, prompt_hi=2)
    assert logits.shape[1] > 2 * 256 + 300
    meta = dict(clip_ratio=0.2, kl_coef=0.001, kl_penalty="low_var_kl", entropy_coeff=0.001)
    zo = logits.float().requires_grad_()
    want, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want, zo)
    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.001), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.001})
    zd = logits.to(dev).requires_grad_()
    got, got_stats = f.compute_loss(zd, _to_dev(b, dev), fused=True, grad_inplace=False, **_to_dev(kw, dev))
    (dz,) = torch.autograd.grad(got, zd)
    assert abs(got.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    for k in want_stats:
        assert abs(got_stats[k] - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    err = (dz.float().cpu() - dz_o).abs().max().item()
    assert err < TOL_DLOGITS and err <= 2 ** -8 * dz_o.abs().max().item() + 1e-9
    # the split kernels on the same batch (persistent backward) agree with the fused sweep
    zs = logits.to(dev).requires_grad_()
    loss_s, _ = f.compute_loss(zs, _to_dev(b, dev), fused=False, **_to_dev(kw, dev))
    (dz_s,) = torch.autograd.grad(loss_s, zs)
    assert loss_s.item() == pytest.approx(got.item(), rel=5e-5)
    assert (dz_s.float() - dz.float()).abs().max().item() <= 2 ** -7 * dz.float().abs().max().item()


@pytest.mark.parametrize("tokens,vocab,hdim", [(300, 1000, 128), (129, 256, 64), (64, 4096 + 24, 256),
                                               (517, 2 * 2048 + 256, 3584)])
def test_lmhead_logprob_forward(dev, tokens, vocab, hdim):
    """Fused lm_head + log-prob on the bf16 matrix cores against F.linear (fp32) + the vocabulary oracle:
    ragged token and vocabulary tiles, labels outside the vocabulary, temperature."""
    gen = torch.Generator().manual_seed(tokens + vocab)
    h = torch.randn(tokens, hdim, generator=gen).to(torch.bfloat16)
    w = (torch.randn(vocab, hdim, generator=gen) * (2.0 / hdim ** 0.5)).to(torch.bfloat16)
    y = torch.randint(0, vocab, (tokens,), generator=gen)
    y[1] = -1
    y[2] = vocab
    for inv_t in (1.0, 1.0 / 0.7):
        lp_o, h_o, lse_o = o_vocab.lmhead_logprob_entropy(h, w, y, inv_t)
        lp, ent, lse = mrl.lmhead_logprob(h.to(dev), w.to(dev), y.to(dev), inv_temperature=inv_t)
        assert lp.shape == (tokens,) and lp.dtype == torch.float32
        assert (lse.cpu() - lse_o).abs().max().item() < 1e-4
        assert (lp.cpu() - lp_o).abs().max().item() < 2e-4
        assert (ent.cpu() - h_o).abs().max().item() < 2e-4
    lp2, ent2, _ = mrl.lmhead_logprob(h.to(dev).view(1, tokens, hdim), w.to(dev), y.to(dev).view(1, tokens).int(),
                                      want_entropy=False)
    assert lp2.shape == (1, tokens) and ent2.abs().sum().item() == 0
    assert torch.allclose(lp2.view(-1).cpu(), o_vocab.lmhead_logprob_entropy(h, w, y)[0], atol=2e-4)


@pytest.mark.parametrize("chunk_rows", [64, 8192])
def test_fused_lmhead_policy_loss(dev, chunk_rows):
    """Loss and gradients straight from the hidden states (per chunk: logits product -> fused sweep ->
    dHidden and dWeight products, all hand-written).  The oracle is fed the bf16 logits that
    mrl_lmhead_logits yields for the same operands (themselves checked against an fp32 product in
    test_lmhead_products_through_the_c_abi), so that the comparison is about everything after the
    rounding of the logits; its dlogits are rounded to bf16 like the pipeline's, and dHidden / dWeight
    are held to 2^-7 of their largest entry (one bf16 rounding of the result plus what single dlogits
    entries that round the other way add up to)."""
    gen = torch.Generator().manual_seed(23)
    vocab, hdim = 2048, 128
    _, b, kw, _, _ = _make_batch(gen, 2, 4, 5, 24, vocab, torch.bfloat16, 1.0, 2)
    total = b["labels"].shape[1]
    h = torch.randn(1, total, hdim, generator=gen).to(torch.bfloat16)
    w = (torch.randn(vocab, hdim, generator=gen) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    hd, wd = h.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    zd = torch.empty(total, vocab, dtype=torch.bfloat16, device=dev)    # what the pipeline's first product yields
    _lib.call("mrl_lmhead_logits", hd.data_ptr(), wd.data_ptr(), total, vocab, hdim, zd.data_ptr(), vocab, _lib.stream(dev))
    logits = zd.cpu()
    meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.002)
    zo = logits.float().view(1, total, vocab).requires_grad_()
    want, want_stats = o_loss.grpo_compute_loss(zo, b, meta, **kw)
    (dz,) = torch.autograd.grad(want, zo)
    dz16 = dz[0].to(torch.bfloat16).float()
    dh_want = dz16 @ w.float()
    dw_want = dz16.t() @ h[0].float()
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    loss, out = mrl.fused_lmhead_policy_loss(hd, wd, bd, packed=True, seqlens=kwd["seqlens_in_batch"],
                                             cu_seqlens=kwd["cu_seqlens_padded"], ref_log_prob=bd["ref_log_prob"],
                                             clip_low=0.2, clip_high=0.2, kl_penalty="low_var_kl", kl_coef=0.01,
                                             entropy_coeff=0.002, chunk_rows=chunk_rows)
    assert abs(loss.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    host = out.cpu().tolist()
    for k, v in zip(("actor/pg_clipfrac", "actor/ppo_kl", "actor/kl_loss", "actor/entropy"), host[2:6]):
        assert abs(v - want_stats[k]) <= TOL_LOSS_REL * abs(want_stats[k]) + 1e-6, k
    dh, dw = torch.autograd.grad(loss * 0.5, [hd, wd])
    assert dh.shape == hd.shape and dw.shape == wd.shape and dh.dtype == torch.bfloat16
    assert (dh.float().cpu()[0] * 2 - dh_want).abs().max().item() <= 2 ** -7 * dh_want.abs().max().item()
    assert (dw.float().cpu() * 2 - dw_want).abs().max().item() <= 2 ** -7 * dw_want.abs().max().item()


@pytest.mark.parametrize("algo", ["grpo", "dapo", "ppo"])
def test_loss_objects_take_hidden_states_and_lm_head_weight(dev, algo):
    """The lm_head path behind the reference's own call surface: the training engine binds everything but
    the model output with functools.partial and Megatron calls loss_func(output), then back-propagates
    loss / num_microbatches (models/base/base_training_engine.py:236-270).  With lm_head_weight= bound
    as well, `output` is the hidden states: same loss and statistics as the oracle on the projected
    logits, and backward() reaches the hidden states and the weight.  The oracle is fed the bf16 logits
    of the pipeline's own first product (one bf16 rounding away from F.linear, asserted here), its
    dlogits are rounded to bf16 like the pipeline's.  Forward-only calls (old / reference log-probs)
    take the same keyword and score the fp32 logits without storing any."""
    from functools import partial
    gen = torch.Generator().manual_seed({"grpo": 41, "dapo": 42, "ppo": 43}[algo])
    vocab, hdim, inv_t = 2048, 128, 1.0 / 0.8
    _, b, kw, _, _ = _make_batch(gen, 2, 4, 5, 24, vocab, torch.bfloat16, 1.0, 2, prompt_hi=6)
    total = b["labels"].shape[1]
    h = torch.randn(1, total, hdim, generator=gen).to(torch.bfloat16)
    w = (torch.randn(vocab, hdim, generator=gen) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    z32 = torch.nn.functional.linear(h[0].float(), w.float())
    # old / reference log-probs around the current policy, as the rollout side would have stored them
    rmask = o_pack.generate_mask(torch.zeros_like(b["advantages"]), b["response_length"])
    lp0 = o_loss.logprob_computer((z32 * inv_t).view(1, total, vocab), b, True, **kw)[0]
    b["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    b["ref_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    hd, wd = h.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    zd = torch.empty(total, vocab, dtype=torch.bfloat16, device=dev)
    _lib.call("mrl_lmhead_logits", hd.data_ptr(), wd.data_ptr(), total, vocab, hdim, zd.data_ptr(), vocab, _lib.stream(dev))
    logits = zd.cpu().float()
    assert (logits - z32).abs().max().item() <= 2 ** -8 * z32.abs().max().item()
    if algo == "grpo":
        meta_o = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.002)
        meta_d = {"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl", "entropy_coeff": 0.002}
        oracle_loss, key = o_loss.grpo_compute_loss, ("ray_grpo", "actor")
    elif algo == "dapo":
        meta_o = dict(clip_ratio=0.2, clip_higher_enable=True, clip_ratio_low=0.2, clip_ratio_high=0.28,
                      token_level_loss=False, entropy_coeff=0.002)
        meta_d = dict(meta_o)
        oracle_loss, key = o_loss.dapo_compute_loss, ("ray_dapo", "actor")
    else:
        meta_o = dict(clip_ratio=0.2, entropy_coeff=0.002)
        meta_d = {"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.0), "entropy_coeff": 0.002}
        oracle_loss, key = o_loss.ppo_compute_loss, ("ray_ppo", "actor")
    zo = logits.view(1, total, vocab).requires_grad_()
    want, want_stats = oracle_loss(zo * inv_t, b, meta_o, **kw)
    (dz,) = torch.autograd.grad(want, zo)
    dz16 = dz[0].to(torch.bfloat16).float()
    n_micro = 4
    dh_want = (dz16 @ w.float()) / n_micro
    dw_want = (dz16.t() @ h[0].float()) / n_micro

    f = mrl.LossFuncFactory.get_instance(*key)
    f.add_loss_meta_info(meta_d)
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    # exactly the caller's steps: bind, call with the model output alone, scale, backward
    loss_func = partial(f.compute_loss, batch=bd, forward_only=False, non_loss_data=True, lm_head_weight=wd,
                        inv_temperature=inv_t, lm_head_chunk_rows=64, **kwd)
    loss, stats = loss_func(hd)
    assert loss.dim() == 0 and loss.requires_grad and all(isinstance(v, float) for v in stats.values())
    (loss / n_micro).backward()
    assert abs(loss.item() - want.item()) <= TOL_LOSS_REL * abs(want.item()) + 1e-7
    assert set(stats) == set(want_stats)
    for k, v in want_stats.items():
        assert abs(stats[k] - v) <= TOL_LOSS_REL * abs(v) + 1e-6, k
    assert hd.grad.shape == hd.shape and wd.grad.shape == wd.shape and hd.grad.dtype == torch.bfloat16
    assert (hd.grad.float().cpu()[0] - dh_want).abs().max().item() <= 2 ** -7 * dh_want.abs().max().item()
    assert (wd.grad.float().cpu() - dw_want).abs().max().item() <= 2 ** -7 * dw_want.abs().max().item()
    # forward only, through the actor object and through the reference-policy object: [B, L] log-probs of
    # the fp32 logits, nothing stored
    want_lp = o_loss.logprob_computer((z32 * inv_t).view(1, total, vocab), b, True, **kw)[0]
    ref_fn = mrl.LossFuncFactory.get_instance("ray_grpo", "reference")
    for obj in (f, ref_fn):
        with torch.no_grad():
            lp = partial(obj.compute_loss, batch=bd, forward_only=True, lm_head_weight=wd.detach(),
                         inv_temperature=inv_t, **kwd)(hd.detach())
        assert lp.shape == want_lp.shape
        assert (lp.cpu() - want_lp).abs().max().item() < 2e-4
    lp_rows, ent_rows = f.compute_log_probs(hd.detach(), bd, skip_entropy=False, lm_head_weight=wd.detach(),
                                            inv_temperature=inv_t, **kwd)
    want_ent = o_loss.logprob_computer((z32 * inv_t).view(1, total, vocab), b, False, **kw)[1]
    assert (ent_rows.cpu() - want_ent).abs().max().item() < 2e-4


@pytest.mark.parametrize("tokens,vocab,hdim", [(517, 4352, 3584), (300, 1000, 128), (64, 4096 + 24, 256), (1, 8, 64),
                                               (777, 2048, 192), (4100, 520, 64)])
def test_lmhead_products_through_the_c_abi(dev, tokens, vocab, hdim):
    """The three matrix products of the lm_head training step, hand-written for the matrix cores:
    logits = hidden W^T (mrl_lmhead_logits), dHidden = dlogits W and dWeight += dlogits^T hidden
    (mrl_lmhead_logprob_bwd), against fp32 products of the same bf16 operands on the CPU: ragged token
    and vocabulary tiles, a vocabulary and token counts that are no multiples of the 64-wide k-step, two
    accumulating calls into one dWeight, untouched padding.  The backward reads hidden, weight and
    dlogits as they lie: memory right behind hidden and weight is filled with NaN to show that rows of k
    beyond the operand are not read."""
    gen = torch.Generator().manual_seed(tokens * 7 + vocab)
    h = torch.randn(tokens, hdim, generator=gen).to(torch.bfloat16)
    w = (torch.randn(vocab, hdim, generator=gen) * (2.0 / hdim ** 0.5)).to(torch.bfloat16)
    dz = (torch.randn(tokens, vocab, generator=gen) * 0.01).to(torch.bfloat16)
    # 64 rows of NaN behind each operand: a k-step that ran past the last row would pick them up
    hbuf = torch.full((tokens + 64, hdim), float("nan"), dtype=torch.bfloat16, device=dev)
    wbuf = torch.full((vocab + 64, hdim), float("nan"), dtype=torch.bfloat16, device=dev)
    hbuf[:tokens] = h.to(dev)
    wbuf[:vocab] = w.to(dev)
    hd, wd = hbuf[:tokens], wbuf[:vocab]
    lib = _lib.load()
    stream = _lib.stream(dev)
    v_pad = (vocab + 63) // 64 * 64
    z = torch.full((tokens, v_pad), 7.0, dtype=torch.bfloat16, device=dev)
    _lib.call("mrl_lmhead_logits", hd.data_ptr(), wd.data_ptr(), tokens, vocab, hdim, z.data_ptr(), v_pad, stream)
    want_z = h.float() @ w.float().t()
    err = (z[:, :vocab].float().cpu() - want_z).abs().max().item()
    assert err <= 2 ** -8 * want_z.abs().max().item() + 1e-6                   # one bf16 rounding of the result
    assert (z[:, vocab:] == 7.0).all().item()                                   # the padding is not written
    # backward: the padding columns of dlogits must be zero; rows behind its last one hold NaN
    dzbuf = torch.full((tokens + 64, v_pad), float("nan"), dtype=torch.bfloat16, device=dev)
    dzbuf[:tokens] = 0
    dzbuf[:tokens, :vocab] = dz.to(dev)
    dzd = dzbuf[:tokens]
    dh = torch.full((tokens, hdim), 5.0, dtype=torch.bfloat16, device=dev)
    dw = torch.ones(vocab, hdim, dtype=torch.float32, device=dev)
    for _ in range(2):                                                           # dWeight accumulates
        _lib.call("mrl_lmhead_logprob_bwd", hd.data_ptr(), wd.data_ptr(), dzd.data_ptr(), v_pad, tokens, vocab, hdim,
                  dh.data_ptr(), dw.data_ptr(), stream)
    want_dh = dz.float() @ w.float()
    want_dw = 1.0 + 2.0 * (dz.float().t() @ h.float())
    assert (dh.float().cpu() - want_dh).abs().max().item() <= 2 ** -7 * want_dh.abs().max().item() + 1e-9
    assert (dw.cpu() - want_dw).abs().max().item() <= 2 ** -7 * (want_dw - 1.0).abs().max().item() + 1e-6
    # rejected shapes: nothing is launched
    assert lib.mrl_lmhead_logits(hd.data_ptr(), wd.data_ptr(), tokens, vocab, hdim - 8, z.data_ptr(), v_pad, stream) == -2
    assert lib.mrl_lmhead_logprob_bwd(hd.data_ptr(), wd.data_ptr(), dzd.data_ptr(), v_pad - 8, tokens, vocab, hdim,
                                      dh.data_ptr(), dw.data_ptr(), stream) == -1
    assert b"dlogits_row_stride" in lib.mrl_last_error()


def test_lmhead_products_random_shapes(dev):
    """40 seeded shapes of the three lm_head products (tokens 1 .. 2500, vocabularies that are multiples of 8
    up to 3000, hidden sizes that are multiples of 64 up to 768: ragged tiles along every dimension, k-steps
    that end inside a tile, single-tile and many-tile grids) against fp32 products on the device; memory
    behind every operand holds NaN."""
    rnd = random.Random(20251)
    lib = _lib.load()
    stream = _lib.stream(dev)
    for case in range(40):
        tokens = rnd.choice([1, 7, 63, 64, 65, 255, 256, 257, 511, 1000, rnd.randint(1, 2500)])
        vocab = 8 * rnd.choice([1, 7, 8, 9, 31, 32, 33, 100, rnd.randint(1, 375)])
        hdim = 64 * rnd.choice([1, 2, 3, 4, 7, 12])
        g = torch.Generator(device=dev).manual_seed(case)
        v_pad = (vocab + 63) // 64 * 64
        hbuf = torch.full((tokens + 64, hdim), float("nan"), dtype=torch.bfloat16, device=dev)
        wbuf = torch.full((vocab + 64, hdim), float("nan"), dtype=torch.bfloat16, device=dev)
        dzbuf = torch.full((tokens + 64, v_pad), float("nan"), dtype=torch.bfloat16, device=dev)
        hbuf[:tokens] = torch.randn(tokens, hdim, generator=g, device=dev).to(torch.bfloat16)
        wbuf[:vocab] = (torch.randn(vocab, hdim, generator=g, device=dev) * (2.0 / hdim ** 0.5)).to(torch.bfloat16)
        dzbuf[:tokens] = 0
        dzbuf[:tokens, :vocab] = (torch.randn(tokens, vocab, generator=g, device=dev) * 0.01).to(torch.bfloat16)
        h, w, dz = hbuf[:tokens], wbuf[:vocab], dzbuf[:tokens]
        what = "case %d: tokens=%d vocab=%d hidden=%d" % (case, tokens, vocab, hdim)
        z = torch.full((tokens, v_pad), 7.0, dtype=torch.bfloat16, device=dev)
        _lib.call("mrl_lmhead_logits", h.data_ptr(), w.data_ptr(), tokens, vocab, hdim, z.data_ptr(), v_pad, stream)
        want = h.float() @ w.float().t()
        assert (z[:, :vocab].float() - want).abs().max().item() <= 2 ** -8 * want.abs().max().item() + 1e-6, what
        assert (z[:, vocab:] == 7.0).all().item(), what
        dh = torch.full((tokens, hdim), 5.0, dtype=torch.bfloat16, device=dev)
        dw = torch.ones(vocab, hdim, dtype=torch.float32, device=dev)
        _lib.call("mrl_lmhead_logprob_bwd", h.data_ptr(), w.data_ptr(), dz.data_ptr(), v_pad, tokens, vocab, hdim,
                  dh.data_ptr(), dw.data_ptr(), stream)
        want_dh = dz[:, :vocab].float() @ w.float()
        want_dw = 1.0 + dz[:, :vocab].float().t() @ h.float()
        assert (dh.float() - want_dh).abs().max().item() <= 2 ** -7 * want_dh.abs().max().item() + 1e-9, what
        assert (dw - want_dw).abs().max().item() <= 1e-5 * (want_dw - 1.0).abs().max().item() + 1e-7, what


def test_copy_kernel_moves_bytes(dev):
    src = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device=dev)
    dst = torch.zeros_like(src)
    _lib.call("mrl_copy_bytes", src.data_ptr(), dst.data_ptr(), src.numel(), _lib.stream(dev))
    assert torch.equal(src, dst)


def test_bandwidth_probes_touch_exactly_their_range(dev):
    """The probes the roofline is quoted against: both copy patterns copy exactly n_rows * row_bytes
    bytes, both write patterns write exactly that many, the read patterns write nothing."""
    rows, row_bytes = 37, 19 * 1024 * 16 - 4096 + 16
    n = rows * row_bytes
    src = torch.randint(0, 255, (n + 64,), dtype=torch.uint8, device=dev)
    for mode in (2, 5):
        dst = torch.full((n + 64,), 7, dtype=torch.uint8, device=dev)
        _lib.call("mrl_bandwidth_probe", mode, src.data_ptr(), dst.data_ptr(), rows, row_bytes, _lib.stream(dev))
        assert torch.equal(dst[:n], src[:n]) and (dst[n:] == 7).all().item()
    for mode in (1, 4):
        dst = torch.full((n + 64,), 7, dtype=torch.uint8, device=dev)
        _lib.call("mrl_bandwidth_probe", mode, 0, dst.data_ptr(), rows, row_bytes, _lib.stream(dev))
        want = torch.tensor([1, 2, 3, 4], dtype=torch.int32).view(torch.uint8).repeat(n // 16).to(dev)
        assert torch.equal(dst[:n], want) and (dst[n:] == 7).all().item()
    for mode in (0, 3):
        sink = torch.full((64,), 7, dtype=torch.uint8, device=dev)
        _lib.call("mrl_bandwidth_probe", mode, src.data_ptr(), sink.data_ptr(), rows, row_bytes, _lib.stream(dev))
        assert (sink == 7).all().item()


def _raw_fused_sweep(z, y, row_ops, dz, ent, terms, stream, ticket=None, scale_dev=None):
    rows, vocab = z.shape
    _lib.call("mrl_fused_logprob_loss", z.data_ptr(), _lib.dtype_code(z), rows, vocab, vocab, y.data_ptr(), _lib.I64,
              1.0, row_ops.data_ptr(), 1, 0.8, 1.2, 3, 0.01, 0.002, 1.0, _lib.ptr(scale_dev), dz.data_ptr(), vocab,
              None, ent.data_ptr(), terms.data_ptr(), _lib.ptr(ticket), 0 if ticket is None else 16, 0, stream)


def _raw_fused_case(dev, seed, rows, vocab):
    gen = torch.Generator().manual_seed(seed)
    z = _logits(gen, rows, vocab, torch.bfloat16).to(dev)
    y = torch.randint(0, vocab, (rows,), generator=gen).to(dev)
    ops = torch.zeros(rows, 8)
    ops[:, 0] = -torch.rand(rows, generator=gen) * 8                   # old log-prob
    ops[:, 1] = -torch.rand(rows, generator=gen) * 8                   # ref log-prob
    ops[:, 2] = torch.randn(rows, generator=gen)                       # advantage
    ops[:, 3] = (torch.rand(rows, generator=gen) > 0.2).float()        # mask: a fifth of the rows is skipped
    ops[:, 4] = 1.0 / rows
    ops[:, 5] = 1.0 / rows
    return z, y, ops.to(dev)


def test_fused_sweep_on_two_streams_and_in_a_graph(dev):
    """The persistent sweep hands out rows through a counter that the caller owns and that a launch
    clears on its own stream: two sweeps in flight on two streams (a counter each), a sweep without a
    counter (one workgroup per row) and a captured sweep replayed several times next to eager sweeps
    (the clearing is a kernel, so it is part of the graph, and the graph keeps its own counter) give
    the results of a lone eager call, bit for bit - every row's result is independent of the order in
    which rows are taken."""
    rows, vocab = 1500, 8200
    cases = [_raw_fused_case(dev, 50 + i, rows, vocab) for i in range(2)]
    tickets = [torch.full((4,), 12345, dtype=torch.int32, device=dev) for _ in range(3)]      # 16-byte workspaces
    want = []
    for z, y, ops in cases:
        dz, ent, terms = torch.empty_like(z), torch.empty(rows, device=dev), torch.empty(rows, 8, device=dev)
        _raw_fused_sweep(z, y, ops, dz, ent, terms, _lib.stream(dev), tickets[0])
        torch.cuda.synchronize()
        want.append((dz, ent, terms))
        assert dz.float().abs().max().item() > 0 and not dz[ops[:, 3] == 0].any().item()
        # every row was handed out exactly once: the workgroups start on the first rows, ticket t stands
        # for row t + workgroups, and each workgroup draws one ticket too many
        assert int(tickets[0][0].item()) == rows
    # no counter: one workgroup per row
    z, y, ops = cases[0]
    plain = (torch.empty_like(z), torch.empty(rows, device=dev), torch.empty(rows, 8, device=dev))
    _raw_fused_sweep(z, y, ops, *plain, _lib.stream(dev), None)
    torch.cuda.synchronize()
    for a, b in zip(plain, want[0]):
        assert torch.equal(a, b)
    # two streams at once, several rounds
    streams = [torch.cuda.Stream(device=dev) for _ in cases]
    outs = [(torch.empty_like(c[0]), torch.empty(rows, device=dev), torch.empty(rows, 8, device=dev)) for c in cases]
    torch.cuda.synchronize()
    for _ in range(4):
        for (z, y, ops), (dz, ent, terms), s, t in zip(cases, outs, streams, tickets):
            _raw_fused_sweep(z, y, ops, dz, ent, terms, s.cuda_stream, t)
    torch.cuda.synchronize()
    for got, ref in zip(outs, want):
        for a, b in zip(got, ref):
            assert torch.equal(a, b)
    # many launches in a row on one stream may share one counter (each clears it behind the previous sweep)
    for _ in range(300):
        _raw_fused_sweep(cases[0][0], cases[0][1], cases[0][2], *outs[0], _lib.stream(dev), tickets[0])
    torch.cuda.synchronize()
    for a, b in zip(outs[0], want[0]):
        assert torch.equal(a, b)
    # captured once, replayed with eager work in between
    z, y, ops = cases[0]
    dz, ent, terms = torch.zeros_like(z), torch.zeros(rows, device=dev), torch.zeros(rows, 8, device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _raw_fused_sweep(z, y, ops, dz, ent, terms, _lib.stream(dev), tickets[2])
    side = torch.cuda.Stream(device=dev)
    for i in range(3):
        dz.zero_()
        ent.zero_()
        terms.zero_()
        other = torch.empty_like(cases[1][0])
        o_ent, o_terms = torch.empty(rows, device=dev), torch.empty(rows, 8, device=dev)
        torch.cuda.synchronize()
        # an eager sweep on another stream runs next to the replay, with a counter of its own
        _raw_fused_sweep(cases[1][0], cases[1][1], cases[1][2], other, o_ent, o_terms, side.cuda_stream, tickets[1])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dz, want[0][0]) and torch.equal(ent, want[0][1]) and torch.equal(terms, want[0][2]), i
        assert torch.equal(other, want[1][0])


@pytest.mark.parametrize("workload", ["c1", "c4chunk", "c2"])
def test_full_size_properties(dev, workload):
    """configs[1] at its full size (128 responses, about 171 k packed rows x 152064 bf16 = 52 GB of
    logits), the same batch as configs[2]'s padded [128, S, 152064] logits (79 GB, with a group of empty
    responses and a group of all-equal rewards) and one 64 k-row chunk of configs[4] (DAPO clip-higher,
    no KL, V = 129280), where the oracle cannot follow: the fused sweep and the split kernels
    (independent code) agree on loss, statistics and dlogits; every dlogits row sums to zero (the
    softmax gradient is orthogonal to the constant vector); rows without a response token (prompt
    rows, padding) are exactly zero; and a random sample of rows matches the oracle's closed forms.
    The split leg writes its gradient over the logits (grad_inplace) so that the padded case fits."""
    import bench
    import gc
    w = bench.WORKLOADS[workload]
    gc.collect()
    torch.cuda.empty_cache()                    # blocks cached by earlier tests count as used otherwise
    free, _ = torch.cuda.mem_get_info(dev)
    if free < {"c1": 190, "c2": 230, "c4chunk": 70}[workload] * 2 ** 30:
        pytest.skip("needs more free HBM")
    plen, rlen, rewards = bench.make_lengths(torch, w, 0)
    logits, b, kw, total = bench.build_device_batch(torch, mrl, w, plen, rlen, rewards, dev, 0)
    vocab = logits.shape[-1]
    flat = logits.view(-1, vocab)
    flat_labels = b["labels"].reshape(-1)
    assert flat.shape[0] == total
    # rows that carry a response token (prompt length 1 everywhere: the first R_i rows of each sequence)
    live = torch.zeros(total, dtype=torch.bool)
    if w.get("layout") == "padded":
        width = logits.shape[1]
        assert logits.shape[0] == 128 and total == 128 * width
        for i, r in enumerate(rlen.flatten().tolist()):
            live[i * width:i * width + r] = True
        assert (rlen.reshape(-1, w["group"]) == 0).all(1).any().item()          # the group of empty responses
    else:
        cu = kw["cu_seqlens_padded"].cpu().tolist()
        for i, r in enumerate(rlen.flatten().tolist()):
            live[cu[i]:cu[i] + r] = True
    live_d = live.to(dev)
    if w.get("loss") == "dapo":
        f = mrl.LossFuncFactory.get_instance("ray_dapo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.2, "clip_higher_enable": True, "clip_ratio_low": 0.2,
                              "clip_ratio_high": 0.28, "token_level_loss": True, "entropy_coeff": 0.001})
    else:
        f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.001), "kl_penalty": "low_var_kl",
                              "entropy_coeff": 0.001})
    # a sample of rows against the oracle: log-prob and entropy (taken first: the split leg below
    # overwrites the logits)
    gen = torch.Generator().manual_seed(5)
    live_idx = torch.nonzero(live).flatten()
    pick = torch.cat([live_idx[torch.randint(0, live_idx.numel(), (40,), generator=gen)],
                      torch.randint(0, total, (8,), generator=gen)])
    pick_d = pick.to(dev)
    zs = flat[pick_d].float().cpu()
    ys = flat_labels[pick_d].cpu()
    lp, h, lse = mrl.vocab_logprob_entropy(flat, flat_labels)
    want_lp = o_vocab.compute_log_probs(zs, ys)
    want_h = o_vocab.vocab_parallel_entropy(zs)
    assert (lp[pick_d].cpu() - want_lp).abs().max().item() < TOL_LOGP
    assert (h[pick_d].cpu() - want_h).abs().max().item() < TOL_LOGP
    del lp, h, lse

    z1 = logits.detach().requires_grad_()
    loss_f, stats_f = f.compute_loss(z1, b, fused=True, **kw)
    (dz_f,) = torch.autograd.grad(loss_f, z1)
    dz_f = dz_f.view(-1, vocab)
    got = dz_f[pick_d].float().cpu()
    z2 = logits.detach().requires_grad_()
    loss_s, stats_s = f.compute_loss(z2, b, fused=False, grad_inplace=True, **kw)
    (dz_s,) = torch.autograd.grad(loss_s, z2)
    dz_s = dz_s.view(-1, vocab)
    assert dz_s.data_ptr() == logits.data_ptr()
    assert loss_s.item() == pytest.approx(loss_f.item(), rel=TOL_LOSS_REL)
    for k in stats_f:
        # ppo_kl is a mean of 171 k differences of about +-0.05 that nearly cancels (5e-6): the absolute
        # term covers the rounding of the log-probs (ulp 1e-6 at -10) in two different summation orders
        assert stats_s[k] == pytest.approx(stats_f[k], rel=TOL_LOSS_REL, abs=2e-6), k
    rows_per = 8192
    scale, worst_sum, worst_diff = 0.0, 0.0, 0.0
    for lo in range(0, total, rows_per):
        a = dz_f[lo:lo + rows_per].float()
        c = dz_s[lo:lo + rows_per].float()
        scale = max(scale, a.abs().max().item())
        worst_diff = max(worst_diff, (a - c).abs().max().item())
        worst_sum = max(worst_sum, a.sum(-1).abs().max().item())
        # rows that are no response token get exactly zero from both paths
        dead = ~live_d[lo:lo + rows_per]
        assert a.abs().amax(-1)[dead].max().item() == 0 if dead.any().item() else True
        assert c.abs().amax(-1)[dead].max().item() == 0 if dead.any().item() else True
        del a, c
    assert scale > 0
    assert worst_diff <= 2 ** -7 * scale
    assert worst_sum <= 0.02 * scale                    # 152 k bf16 roundings against a one-hot entry of `scale`
    assert (~live).sum().item() >= rlen.numel()
    # dlogits of a live row is c0 * (onehot - p) - c1 * p * (z - E z): recover c0 from the label entry and
    # check the rest of the row against the oracle's softmax with it (entropy coefficient folded into c1)
    p = torch.softmax(zs, -1)
    ent_term = p * (zs - (p * zs).sum(-1, keepdim=True))
    onehot = torch.zeros_like(p)
    onehot[torch.arange(len(ys)), ys] = 1.0
    basis0, basis1 = onehot - p, -ent_term
    checked = 0
    for i in range(len(pick)):
        assert bool(got[i].any()) == bool(live[pick[i]]) or not live[pick[i]]
        if not got[i].any():
            continue
        a = torch.stack([basis0[i], basis1[i]], 1).double()
        coef = torch.linalg.lstsq(a, got[i].double().unsqueeze(1)).solution
        resid = (a @ coef).squeeze(1) - got[i].double()
        assert resid.abs().max().item() <= 2 ** -8 * got[i].abs().max().item() + 1e-12, i
        checked += 1
    assert checked >= 30


def test_full_size_lmhead_forward(dev):
    """configs[3]'s forward at its full size (163 840 tokens x 3584 hidden x 152 064 vocabulary, logits
    never stored): 48 sampled tokens against the oracle (fp32 product of the bf16 operands on the CPU),
    4096 tokens against an fp32 GEMM + log-softmax on the device, and size-independent properties over
    all tokens: 0 <= entropy <= ln V, logp <= 0, logsumexp finite, and the static-scratch entry
    point's limit respected by slicing."""
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 40 * 2 ** 30:
        pytest.skip("needs more free HBM")
    tokens, vocab, hdim = 163840, 152064, 3584
    g = torch.Generator(device=dev).manual_seed(3)
    hidden = torch.randn(tokens, hdim, generator=g, device=dev).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (tokens,), generator=g, device=dev)
    lp, ent, lse = mrl.lmhead_logprob(hidden, weight, labels, inv_temperature=1.0)
    torch.cuda.synchronize()
    assert torch.isfinite(lse).all().item() and (lp <= 0).all().item()
    assert (ent >= 0).all().item() and (ent <= math.log(vocab) + 1e-3).all().item()
    gen = torch.Generator().manual_seed(4)
    pick = torch.randint(0, tokens, (48,), generator=gen)
    pick[0], pick[1] = 0, tokens - 1
    lp_o, h_o, lse_o = o_vocab.lmhead_logprob_entropy(hidden[pick.to(dev)].cpu(), weight.cpu(), labels[pick.to(dev)].cpu())
    assert (lse[pick.to(dev)].cpu() - lse_o).abs().max().item() < 1e-4
    assert (lp[pick.to(dev)].cpu() - lp_o).abs().max().item() < 2e-4
    assert (ent[pick.to(dev)].cpu() - h_o).abs().max().item() < 2e-4
    # a contiguous block straddling token tiles, fp32 on the device
    lo = 163840 - 4096 - 77
    ref = torch.log_softmax(torch.nn.functional.linear(hidden[lo:lo + 4096].float(), weight.float()), -1)
    assert (lp[lo:lo + 4096] - ref.gather(-1, labels[lo:lo + 4096, None])[:, 0]).abs().max().item() < 2e-4
    assert (ent[lo:lo + 4096] + (ref.exp() * ref).sum(-1)).abs().max().item() < 2e-4
    del ref
    # the same tokens through the entry point that allocates nothing, in slices of its limit
    lib = _lib.load()
    limit = lib.mrl_lmhead_static_max_tokens()
    lp2, ent2, lse2 = (torch.empty_like(lp) for _ in range(3))
    for c0 in range(0, tokens, limit):
        n = min(limit, tokens - c0)
        _lib.call("mrl_lmhead_logprob_fwd_static", hidden.data_ptr() + c0 * hdim * 2, weight.data_ptr(), n, vocab, hdim,
                  labels.data_ptr() + c0 * 8, _lib.I64, 1.0, lp2.data_ptr() + c0 * 4, ent2.data_ptr() + c0 * 4,
                  lse2.data_ptr() + c0 * 4, _lib.stream(dev))
    torch.cuda.synchronize()
    # the partial statistics of a token do not depend on which other tokens share the call
    assert torch.equal(lp2, lp) and torch.equal(ent2, ent) and torch.equal(lse2, lse)


def test_full_size_lmhead_training_step(dev):
    """configs[3]'s training step at its full size (128 sequences, ~164 k tokens, H = 3584, V = 152 064):
    the step run twice gives bit-identical results; with two different chunkings (32 768 rows, and 20 000
    rows, which is no multiple of a tile) it gives the same loss and the same dHidden bit for bit and the same dWeight up to how fp32 sums group;
    <dWeight, W> = <dHidden, hidden> (both equal sum dlogits * logits: an identity between the two
    backward products that needs no dlogits); and the rows of one whole sequence against the oracle's
    loss gradient (CPU, fed the device's bf16 logits of those rows, scaled by its share of the tokens)
    pushed through an fp32 product with W."""
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 60 * 2 ** 30:
        pytest.skip("needs more free HBM")
    vocab, hdim, n_seq, group = 152064, 3584, 128, 8
    gen = torch.Generator().manual_seed(11)
    rlen = torch.randint(512, 2049, (n_seq,), generator=gen)
    rlen[5] = 300                                              # the sequence the oracle takes
    plen = torch.ones(n_seq, dtype=torch.int64)
    seqlens = (plen + rlen).to(torch.int32)
    cu = torch.zeros(n_seq + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(seqlens, 0)
    total, resp_w, n_tok = int(cu[-1]), int(rlen.max()), int(rlen.sum())
    g = torch.Generator(device=dev).manual_seed(12)
    hidden = torch.randn(1, total, hdim, generator=g, device=dev).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (1, total), generator=g, device=dev)
    rewards = torch.randn(n_seq, 1, generator=gen)
    b = {"labels": labels, "responses": torch.zeros(n_seq, resp_w, dtype=torch.int32, device=dev),
         "response_length": rlen.view(-1, 1).to(dev), "prompt_length": plen.view(-1, 1).to(dev)}
    seqlens_d, cu_d = seqlens.to(dev), cu.to(dev)
    rmask = mrl.generate_mask(b["responses"], b["response_length"])
    b["advantages"], _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), rmask, b["response_length"], group)
    lp_rows, _, _ = mrl.lmhead_logprob(hidden, weight, labels, want_entropy=False)
    lp0 = mrl.postprocess_packed_seqs(lp_rows, seqlens_d, cu_d, resp_w, prompt_length=b["prompt_length"])
    maskf = rmask.to(torch.float32)
    b["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=g, device=dev) * 0.05) * maskf
    ref_lp = (lp0 + torch.randn(lp0.shape, generator=g, device=dev) * 0.05) * maskf
    kl_coef, ent_coef = 0.001, 0.001

    def step(chunk_rows):
        h, wt = hidden.detach().requires_grad_(), weight.detach().requires_grad_()
        loss, out = mrl.fused_lmhead_policy_loss(h, wt, b, packed=True, seqlens=seqlens_d, cu_seqlens=cu_d,
                                                 ref_log_prob=ref_lp, clip_low=0.2, clip_high=0.2, kl_penalty="low_var_kl",
                                                 kl_coef=kl_coef, entropy_coeff=ent_coef, chunk_rows=chunk_rows)
        dh, dw = torch.autograd.grad(loss, [h, wt])
        return loss.item(), out.cpu(), dh[0], dw

    l1, o1, dh1, dw1 = step(32768)
    l1b, o1b, dh1b, dw1b = step(32768)
    # nothing in the step depends on timing: no atomics, dWeight accumulated in stream order
    assert l1b == l1 and torch.equal(o1b, o1) and torch.equal(dh1b, dh1) and torch.equal(dw1b, dw1)
    del dh1b, dw1b
    l2, o2, dh2, dw2 = step(20000)
    assert l1 == l2 and torch.equal(o1, o2)
    assert torch.equal(dh1, dh2)
    dw_max = dw1.float().abs().max().item()
    assert dw_max > 0 and (dw1.float() - dw2.float()).abs().max().item() <= 2 ** -7 * dw_max
    del dh2, dw2
    # the identity between the two backward products
    lhs = (dw1.double() * weight.double()).sum().item()
    rhs = (dh1.double() * hidden[0].double()).sum().item()
    scale = (dw1.double() * weight.double()).abs().sum().item() + (dh1.double() * hidden[0].double()).abs().sum().item()
    assert math.isfinite(lhs) and scale > 0 and abs(lhs - rhs) <= 1e-4 * scale, (lhs, rhs, scale)
    # one whole sequence against the oracle
    s = 5
    r0, r1 = int(cu[s]), int(cu[s + 1])
    rows = r1 - r0
    z = torch.empty(rows, vocab, dtype=torch.bfloat16, device=dev)
    _lib.call("mrl_lmhead_logits", hidden.data_ptr() + r0 * hdim * 2, weight.data_ptr(), rows, vocab, hdim, z.data_ptr(),
              vocab, _lib.stream(dev))
    rl = int(rlen[s])
    ob = {"labels": labels[:, r0:r1].cpu(), "responses": torch.zeros(1, rl, dtype=torch.int32),
          "response_length": rlen[s].view(1, 1), "prompt_length": plen[s].view(1, 1),
          "advantages": b["advantages"][s:s + 1, :rl].cpu(), "old_log_prob": b["old_log_prob"][s:s + 1, :rl].cpu(),
          "ref_log_prob": ref_lp[s:s + 1, :rl].cpu()}
    okw = dict(forward_only=False, use_remove_padding=True, seqlens_in_batch=seqlens[s:s + 1],
               cu_seqlens_padded=torch.tensor([0, rows], dtype=torch.int32), seq_len=rows)
    zo = z.float().cpu().view(1, rows, vocab).requires_grad_()
    meta = dict(clip_ratio=0.2, kl_coef=kl_coef, kl_penalty="low_var_kl", entropy_coeff=ent_coef)
    want, _ = o_loss.grpo_compute_loss(zo, ob, meta, **okw)
    (dz,) = torch.autograd.grad(want, zo)
    dz16 = (dz[0] * (rl / n_tok)).to(torch.bfloat16).to(dev).float()
    dh_want = dz16 @ weight.float()
    got = dh1[r0:r1].float()
    assert (got - dh_want).abs().max().item() <= 2 ** -7 * dh_want.abs().max().item()
    assert dh_want.abs().max().item() > 0


def _random_fused_case(i, rnd):
    """One random case of the raw fused sweep against an fp32 torch chain on the device; returns a
    description of the mismatch or None."""
    dts = {torch.bfloat16: 8, torch.float16: 8, torch.float32: 4}
    dtype = rnd.choice(list(dts))
    per = dts[dtype]
    max_vec = 19 * 1024
    nvec = rnd.choice([rnd.randint(1, 64), rnd.randint(1, max_vec),
                       rnd.choice([1024 * k + d for k in (4, 8, 12, 16, 19) for d in (-1, 0, 1)])])
    nvec = max(1, min(nvec, max_vec))
    rows = rnd.choice([1, 3, 257, 511, 513, 600, 777, 1100])
    if i % 6 == 5:
        # a row that two workgroups hold: between one and two register files wide
        nvec = rnd.choice([max_vec + 1, 2 * max_vec, 2 * max_vec - 1, rnd.randint(max_vec + 1, 2 * max_vec),
                           2 * 1024 * rnd.choice([10, 12, 13, 16]) + rnd.choice([-1, 0, 1])])
        rows = rnd.choice([1, 2, 129, 300, 515])
    vocab = nvec * per
    inv_t = rnd.choice([1.0, 0.7, 1.3])
    ent_c = rnd.choice([0.0, 0.003])
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(i)
    z = (torch.randn(rows, vocab, generator=g, device=dev) * 3).to(dtype)
    y = torch.randint(0, vocab, (rows,), generator=g, device=dev)
    if rows > 2:
        y[1] = -100
        y[2] = vocab + 3
    ops = torch.zeros(rows, 8, device=dev)
    ops[:, 0] = -torch.rand(rows, generator=g, device=dev) * 8
    ops[:, 1] = -torch.rand(rows, generator=g, device=dev) * 8
    ops[:, 2] = torch.randn(rows, generator=g, device=dev)
    ops[:, 3] = (torch.rand(rows, generator=g, device=dev) > 0.25).float()
    ops[:, 4] = 1.0 / rows
    ops[:, 5] = 1.0 / rows
    dz = torch.full_like(z, 7.0)
    ent = torch.zeros(rows, device=dev)
    lp = torch.zeros(rows, device=dev)
    terms = torch.zeros(rows, 8, device=dev)
    # every other narrow case gets no workspace (one workgroup per row whatever the batch); wide rows need theirs
    ws_bytes = _lib.load().mrl_fused_workspace_bytes(_lib.dtype_code(z), rows, vocab)
    assert ws_bytes >= 16
    workspace = torch.full((ws_bytes,), 0xAB, dtype=torch.uint8, device=dev) if (i % 2 == 0 or ws_bytes > 16) else None
    clip_lo, clip_hi, kl_kind, kl_coef = 0.8, 1.25, 4, 0.01
    _lib.call("mrl_fused_logprob_loss", z.data_ptr(), _lib.dtype_code(z), rows, vocab, vocab, y.data_ptr(), _lib.I64,
              inv_t, ops.data_ptr(), 1, clip_lo, clip_hi, kl_kind, kl_coef, ent_c, 1.0, None, dz.data_ptr(), vocab,
              lp.data_ptr(), ent.data_ptr() if ent_c != 0 else None, terms.data_ptr(),
              _lib.ptr(workspace), ws_bytes if workspace is not None else 0, 0, _lib.stream(dev))
    zr = (z.float() * inv_t).requires_grad_()
    logsm = torch.log_softmax(zr, -1)
    y_ok = (y >= 0) & (y < vocab)
    yc = y.clamp(0, vocab - 1)
    # a label outside the vocabulary scores the row maximum and has no one-hot term (Megatron's masked gather)
    lp_ref = torch.where(y_ok, logsm.gather(-1, yc[:, None])[:, 0], zr.max(-1).values.detach() - torch.logsumexp(zr, -1))
    p = logsm.exp()
    h_ref = -(p * logsm).sum(-1)
    old, ref, adv, m, wpg, invtok = [ops[:, k] for k in range(6)]
    ratio = torch.exp(lp_ref - old)
    pg = torch.maximum(-adv * ratio, -adv * ratio.clamp(clip_lo, clip_hi))
    c = (ref - lp_ref).clamp(-20, 20)
    k3 = (torch.exp(c) - c - 1).clamp(-10, 10)
    loss = (pg * m * wpg).sum() + kl_coef * (k3 * m * invtok).sum() - ent_c * (h_ref * m * invtok).sum()
    (g_ref,) = torch.autograd.grad(loss, zr)
    g_ref = g_ref * inv_t
    live = m != 0
    e_lp = (lp[live] - lp_ref.detach()[live]).abs().max().item() if live.any() else 0.0
    scale = g_ref.abs().max().item() + 1e-12
    err = (dz.float() - g_ref).abs().max().item()
    rel = 2 ** -7 if dtype != torch.float32 else 2e-5
    # fp16 gradients below 6.1e-5 are subnormal: their spacing is 2^-24 whatever their size
    floor = 2 ** -25 if dtype == torch.float16 else 1e-9
    ok = e_lp < 2e-4 and err <= rel * scale + floor and not dz[~live].any().item()
    if ent_c != 0 and live.any():
        ok = ok and (ent[live] - h_ref.detach()[live]).abs().max().item() < 2e-4
    return None if ok else (i, dtype, rows, vocab, inv_t, ent_c, e_lp, err, scale)


def test_fused_sweep_random_shapes(dev):
    """Randomised differential test of the fused sweep (all three logits dtypes, row lengths around
    every register-tile boundary, one-row to persistent batches, temperature, entropy on and off,
    skipped rows, labels outside the vocabulary) against an fp32 torch chain on the device."""
    import random
    rnd = random.Random(1234)
    failures = [f for f in (_random_fused_case(i, rnd) for i in range(60)) if f is not None]
    assert not failures, failures


def _random_split_case(i, rnd):
    """One random case of the split forward + backward against an fp32 torch chain on the device."""
    dev = torch.device("cuda:0")
    dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
    vocab = rnd.choice([rnd.randint(1, 300), rnd.randint(300, 40000), rnd.choice([8192, 8200, 16384, 32000, 129280, 152064]),
                        rnd.randint(1, 2500) * 8 + rnd.choice([0, 0, 1, 3, 5])])
    rows = rnd.choice([1, 2, 17, 300, 700])
    if rows * vocab > 60_000_000:
        rows = max(1, 60_000_000 // vocab)
    inv_t = rnd.choice([1.0, 0.5, 1.7])
    pad = rnd.choice([0, 0, 8, 24])
    g = torch.Generator(device=dev).manual_seed(1000 + i)
    wide = (torch.randn(rows, vocab + pad, generator=g, device=dev) * 3).to(dtype)
    z = wide[:, :vocab] if pad else wide
    y = torch.randint(0, vocab, (rows,), generator=g, device=dev)
    if rows > 2:
        y[0] = -100
        y[1] = vocab
    g_lp = torch.randn(rows, generator=g, device=dev) * 0.1
    g_h = torch.randn(rows, generator=g, device=dev) * 0.01
    mode = rnd.choice(["both", "lp", "h"])
    if rows > 2:
        g_lp[2] = 0.0
        g_h[2] = 0.0
    zd = z.detach().requires_grad_()
    lp, h, lse = mrl.vocab_logprob_entropy(zd, y, inv_temperature=inv_t)
    outs, gs = [], []
    if mode in ("both", "lp"):
        outs.append(lp); gs.append(g_lp)
    if mode in ("both", "h"):
        outs.append(h); gs.append(g_h)
    (dz,) = torch.autograd.grad(outs, zd, gs)
    zr = (z.float() * inv_t).requires_grad_()
    logsm = torch.log_softmax(zr, -1)
    y_ok = (y >= 0) & (y < vocab)
    yc = y.clamp(0, vocab - 1)
    lp_ref = torch.where(y_ok, logsm.gather(-1, yc[:, None])[:, 0], zr.max(-1).values.detach() - torch.logsumexp(zr, -1))
    h_ref = -(logsm.exp() * logsm).sum(-1)
    tot = 0
    if mode in ("both", "lp"):
        tot = tot + (lp_ref * g_lp).sum()
    if mode in ("both", "h"):
        tot = tot + (h_ref * g_h).sum()
    (g_ref,) = torch.autograd.grad(tot, zr)
    g_ref = g_ref * inv_t
    e_lp = (lp - lp_ref.detach()).abs().max().item()
    e_h = (h - h_ref.detach()).abs().max().item()
    scale = g_ref.abs().max().item() + 1e-12
    err = (dz.float() - g_ref).abs().max().item()
    rel = 2 ** -7 if dtype != torch.float32 else 3e-5
    floor = 2 ** -25 if dtype == torch.float16 else 1e-9     # the spacing of fp16 subnormals is 2^-24
    ok = e_lp < 2e-4 and e_h < 2e-4 and err <= rel * scale + floor and dz.dtype == dtype and dz.shape == z.shape
    if rows > 2 and mode == "both":
        ok = ok and not dz[2].any().item()
    return None if ok else (i, dtype, rows, vocab, pad, inv_t, mode, e_lp, e_h, err, scale)


def test_split_sweeps_random_shapes(dev):
    """Randomised differential test of the split forward and backward (all logits dtypes, vocabularies
    from 1 to 152064 including sizes that are no multiple of a vector, rows inside a wider buffer,
    temperature, either gradient alone, rows without gradient, labels outside the vocabulary)."""
    import random
    rnd = random.Random(99)
    failures = [f for f in (_random_split_case(i, rnd) for i in range(80)) if f is not None]
    assert not failures, failures


def _random_loss_case(i, rnd, dev):
    """One random actor-loss case end to end against the oracle; returns a description of the mismatch or None."""
    gen = torch.Generator().manual_seed(5000 + i)
    n_prompts, group = rnd.randint(1, 4), rnd.randint(2, 5)
    r_lo = rnd.randint(1, 12); r_hi = r_lo + rnd.randint(0, 40)
    vocab = rnd.choice([64, 1000, 4096])
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    align = rnd.choice([1, 2, 8])
    logits, b, kw, rewards, (ids, labels, mask1d) = _make_batch(gen, n_prompts, group, r_lo, r_hi, vocab, dtype, 2.5, align, prompt_hi=rnd.randint(1, 5))
    batch = ids.shape[0]
    if rnd.random() < 0.5:
        k = rnd.randrange(batch)
        b["response_length"][k] = 0
    kind = rnd.choice(["grpo", "dapo_tok", "dapo_seq", "ppo"])
    fused = rnd.random() < 0.5
    ent = rnd.choice([0.0, 0.002])
    layout = rnd.choice(["packed", "padded"])
    if kind == "grpo":
        meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty=rnd.choice(["low_var_kl", "kl", "abs", "mse"]), entropy_coeff=ent)
        f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": meta["kl_penalty"], "entropy_coeff": ent})
        ofn = o_loss.grpo_compute_loss
    elif kind.startswith("dapo"):
        tok = kind == "dapo_tok"
        if not tok:
            b["response_length"] = torch.clamp(b["response_length"], min=1)     # an all-masked row is NaN in the reference
        meta = dict(entropy_coeff=ent, token_level_loss=tok, clip_higher_enable=True, clip_ratio_low=0.2, clip_ratio_high=0.28)
        f = mrl.LossFuncFactory.get_instance("ray_dapo", "actor")
        f.add_loss_meta_info(dict(meta, clip_ratio=0.2))
        ofn = o_loss.dapo_compute_loss
    else:
        meta = dict(clip_ratio=0.25, entropy_coeff=ent)
        f = mrl.LossFuncFactory.get_instance("ray_ppo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.25, "entropy_coeff": ent, "kl_ctrl": mrl.FixedKLController(0.1)})
        ofn = o_loss.ppo_compute_loss
    zo = logits.float().requires_grad_()
    want, want_stats = ofn(zo, b, meta, **kw)
    (dz_o,) = torch.autograd.grad(want, zo)
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    if layout == "packed":
        zd = logits.to(dev).requires_grad_()
        got, stats = f.compute_loss(zd, bd, fused=fused, **kwd)
        (dz,) = torch.autograd.grad(got, zd)
        dz_cmp = dz.float().cpu()
    else:
        seqlens, cu = kw["seqlens_in_batch"], kw["cu_seqlens_padded"]
        width = ids.shape[1]
        padded = torch.randn(batch, width, vocab, generator=gen).to(dtype)
        for k in range(batch):
            padded[k, :seqlens[k]] = logits[0, cu[k]:cu[k] + seqlens[k]]
        zd = padded.to(dev).requires_grad_()
        got, stats = f.compute_loss(zd, dict(bd, labels=labels.to(dev)), fused=fused)
        (dzp,) = torch.autograd.grad(got, zd)
        dz_cmp = torch.zeros_like(dz_o)
        for k in range(batch):
            dz_cmp[0, cu[k]:cu[k] + seqlens[k]] = dzp[k, :seqlens[k]].float().cpu()
            if dzp[k, seqlens[k]:].any().item():
                return (i, "padding rows not zero")
    # the loss is a mean of terms of size ~1 that may cancel: a few fp32 ulps of 1 remain whatever its size
    tol_l = 1e-4 * abs(want.item()) + 1e-6
    if not abs(got.item() - want.item()) <= tol_l:
        return (i, kind, fused, layout, "loss", got.item(), want.item())
    for k in want_stats:
        if not abs(stats[k] - want_stats[k]) <= 1e-4 * abs(want_stats[k]) + 2e-6:
            return (i, kind, fused, layout, k, stats[k], want_stats[k])
    scale = dz_o.abs().max().item()
    err = (dz_cmp - dz_o).abs().max().item()
    rel = 2 ** -7 if dtype == torch.bfloat16 else 1e-4
    if not err <= rel * scale + 1e-9:
        return (i, kind, fused, layout, dtype, "dlogits", err, scale)
    return None


def test_actor_losses_random_batches(dev):
    """Randomised end-to-end test against the oracle: GRPO with each KL estimator, DAPO token-level and
    sequence-mean, PPO; fused sweep and split kernels; packed (alignment 1, 2, 8) and padded layout with
    noise in the padding rows; fp32 and bf16 logits; empty responses; entropy bonus on and off."""
    import random
    rnd = random.Random(7)
    failures = [f for f in (_random_loss_case(i, rnd, dev) for i in range(80)) if f is not None]
    assert not failures, failures


def _random_index_case(i, rnd, dev):
    """One random case of the mask / pack / unpack / window maps against the oracle, bit for bit."""
    gen = torch.Generator().manual_seed(9000 + i)
    batch = rnd.choice([1, 2, 5, 33, 70])
    width = rnd.choice([1, 2, 7, 64, 131, 200])
    align = rnd.choice([1, 2, 4, 8, 16, 64])
    id_dtype = rnd.choice([torch.int64, torch.int32])
    lens = torch.randint(0, width + 1, (batch, 1), generator=gen, dtype=torch.int32)
    if rnd.random() < 0.3:
        lens[rnd.randrange(batch)] = width
    if rnd.random() < 0.3:
        lens[rnd.randrange(batch)] = 0
    plen = torch.minimum(torch.randint(1, 6, (batch, 1), generator=gen, dtype=torch.int32), torch.clamp(lens, min=1))
    ids = torch.randint(1, 50000, (batch, width), generator=gen).to(id_dtype)
    labels = torch.randint(1, 50000, (batch, width), generator=gen).to(id_dtype)
    mask_o = o_pack.generate_mask(ids, lens)
    mask = mrl.generate_mask(ids.to(dev), lens.to(dev))
    if not (mask.dtype == mask_o.dtype and torch.equal(mask.cpu(), mask_o)):
        return (i, "generate_mask")
    want = o_pack.preprocess_packed_seqs(ids, labels, mask_o, align)
    got = mrl.preprocess_packed_seqs(ids.to(dev), labels.to(dev), mask, align)
    for k, (a, b) in enumerate(zip(got, want)):
        if not (a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.cpu(), b)):
            return (i, "preprocess", k, batch, width, align)
    seqlens, cu = got[3], got[4]
    total = want[0].shape[1]
    resp_w = rnd.choice([max(1, int(lens.max())), width, width + 3])
    for trailing in ((), (3,)):
        packed = torch.randn((1, total) + trailing, generator=gen)
        for prompt in (None, plen):
            seq_len = resp_w if prompt is not None else width
            w = o_pack.postprocess_packed_seqs(packed, want[3], want[4], seq_len, prompt)
            g = mrl.postprocess_packed_seqs(packed.to(dev), seqlens, cu, seq_len, None if prompt is None else prompt.to(dev))
            if not torch.equal(g.cpu(), w):
                return (i, "postprocess", trailing, prompt is not None, batch, width, align, resp_w)
    # padded-layout windows
    rlen = torch.clamp(lens - plen, min=0)
    window = o_pack.response_window(plen, rlen)
    responses = torch.zeros(batch, resp_w)
    x2 = torch.randn(batch, width, generator=gen)
    x3 = torch.randn(batch, width, 5, generator=gen)
    w2 = o_pack.truncate_prompt_and_pad(responses, x2, window)
    g2 = mrl.truncate_prompt_and_pad(responses.to(dev), x2.to(dev), mrl.response_window(plen.to(dev), rlen.to(dev)))
    if not torch.equal(g2.cpu(), w2):
        return (i, "truncate_prompt_and_pad", batch, width, resp_w)
    w3 = o_pack.truncate_middle_and_pad(responses, x3, window)
    g3 = mrl.truncate_middle_and_pad(responses.to(dev), x3.to(dev), mrl.response_window(plen.to(dev), rlen.to(dev)))
    if not torch.equal(g3.cpu(), w3):
        return (i, "truncate_middle_and_pad", batch, width, resp_w)
    return None


def test_index_maps_random_shapes_bit_exact(dev):
    """Randomised bit-exact test of generate_mask, preprocess_packed_seqs (all five outputs),
    postprocess_packed_seqs (with and without the prompt shift, with a trailing dimension) and the
    padded-layout windows: batch 1..70, width 1..200, alignment 1..64, int32 / int64 ids, empty and
    full-width sequences."""
    import random
    rnd = random.Random(3)
    failures = [f for f in (_random_index_case(i, rnd, dev) for i in range(120)) if f is not None]
    assert not failures, failures


def _random_wire_and_gae_case(i, rnd, dev):
    """One random case of the experience wire format and of the GAE scan against the oracle."""
    gen = torch.Generator().manual_seed(400 + i)
    batch = rnd.choice([1, 2, 9, 64, 130])
    hi = rnd.choice([2, 17, 300])
    lens_a = torch.randint(0, hi, (batch,), generator=gen, dtype=torch.int32)
    if int(lens_a.sum()) == 0:
        lens_a[0] = 1
    lens_b = torch.randint(1, 9, (batch,), generator=gen, dtype=torch.int32)
    data = {"responses": torch.randint(0, 1000, (int(lens_a.sum()),), generator=gen),
            "old_log_prob": torch.randn(int(lens_a.sum()), generator=gen),
            "position_ids": torch.randint(0, 99, (3, int(lens_b.sum())), generator=gen),
            "response_length": lens_a.clone()}
    lens = {"responses": lens_a, "old_log_prob": lens_a, "position_ids": lens_b, "response_length": torch.ones(batch, dtype=torch.int32)}
    multiple = rnd.choice([1, 2, 8, 16])
    want = o_pack.unpack_pad_experience(data, lens, -7, multiple)
    got = mrl.unpack_pad_experience({k: v.to(dev) for k, v in data.items()}, lens, -7, multiple)
    for k in want:
        if not (got[k].dtype == want[k].dtype and got[k].shape == want[k].shape and torch.equal(got[k].cpu(), want[k])):
            return (i, "unpack", k, batch, hi, multiple)
    width = rnd.choice([1, 5, 40, 257])
    tensor = torch.randint(0, 500, (batch, width), generator=gen)
    idx = torch.randint(0, width + 1, (batch, 1), generator=gen)
    for left in (False, True):
        w = o_pack.truncate_rows(tensor, idx, left)
        g = mrl.truncate_rows(tensor.to(dev), idx.to(dev), left)
        if len(w) != len(g) or not all(a.dtype == b.dtype and torch.equal(a.cpu(), b) for a, b in zip(g, w)):
            return (i, "truncate_rows", left, batch, width)
    # GAE + whitening
    L = rnd.choice([1, 2, 33, 500, 2100])
    r = torch.randn(batch, L, generator=gen); v = torch.randn(batch, L, generator=gen)
    ml = torch.randint(0, L + 1, (batch,), generator=gen)
    ml[0] = L
    if batch > 1: ml[1] = max(1, L // 2)
    mask = o_pack.generate_mask(torch.zeros(batch, L), ml)
    if int(mask.sum()) < 2:
        return None
    gamma, lam = rnd.choice([(1.0, 0.95), (0.99, 1.0), (0.9, 0.5)])
    wa, wr = o_adv.compute_gae_advantage_return(r, v, mask, torch.tensor(gamma), torch.tensor(lam))
    ga, gr = mrl.compute_gae_advantage_return(r.to(dev), v.to(dev), mask.to(dev), gamma, lam)
    if not torch.equal(gr.cpu(), wr):
        return (i, "gae returns", batch, L, gamma, lam, (gr.cpu() - wr).abs().max().item())
    if not (ga.cpu() - wa).abs().max().item() <= 2e-5 * max(1.0, wa.abs().max().item()):
        return (i, "gae adv", batch, L, (ga.cpu() - wa).abs().max().item())
    return None


def test_wire_format_and_gae_random_shapes(dev):
    """Randomised test of unpack_pad_experience and truncate_rows (bit-exact) and of the GAE scan
    (returns bit-exact, also for rows longer than one staged chunk) against the oracle."""
    import random
    rnd = random.Random(11)
    failures = [f for f in (_random_wire_and_gae_case(i, rnd, dev) for i in range(60)) if f is not None]
    assert not failures, failures


def _random_lmhead_case(i, rnd, dev):
    """One random case of the fused lm_head forward against an fp32 matmul + log-softmax on the device."""
    g = torch.Generator(device=dev).manual_seed(70 + i)
    tokens = rnd.choice([1, 2, 63, 64, 65, 255, 256, 257, 300, 511, 513, 1000])
    vocab = rnd.choice([8, 16, 248, 256, 264, 2040, 2048, 2056, 4096 + 24, 5000, 12345 // 8 * 8, 40000])
    hdim = rnd.choice([64, 128, 192, 256, 1024, 3584])
    inv_t = rnd.choice([1.0, 0.6, 1.5])
    h = torch.randn(tokens, hdim, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(vocab, hdim, generator=g, device=dev) * (2.0 / hdim ** 0.5)).to(torch.bfloat16)
    y = torch.randint(0, vocab, (tokens,), generator=g, device=dev)
    if tokens > 2:
        y[1] = -1
        y[2] = vocab
    want_ent = rnd.random() < 0.7
    lp, ent, lse = mrl.lmhead_logprob(h, w, y, inv_temperature=inv_t, want_entropy=want_ent)
    z = (h.float() @ w.float().t()) * inv_t
    logsm = torch.log_softmax(z, -1)
    y_ok = (y >= 0) & (y < vocab)
    lp_ref = torch.where(y_ok, logsm.gather(-1, y.clamp(0, vocab - 1)[:, None])[:, 0], z.max(-1).values - torch.logsumexp(z, -1))
    h_ref = -(logsm.exp() * logsm).sum(-1)
    e1 = (lp - lp_ref).abs().max().item()
    e2 = (lse - torch.logsumexp(z, -1)).abs().max().item()
    e3 = (ent - h_ref).abs().max().item() if want_ent else ent.abs().max().item()
    ok = e1 < 3e-4 and e2 < 2e-4 and e3 < 3e-4
    return None if ok else (i, tokens, vocab, hdim, inv_t, want_ent, e1, e2, e3)


def test_lmhead_forward_random_shapes(dev):
    """Randomised test of the fused lm_head forward: token counts around the 64- and 256-token tiles,
    vocabularies whose last 256-row tile holds 8 .. 248 rows and is the only tile of its group (a lane
    that never sees a valid row must contribute exactly nothing), hidden sizes 64 .. 3584."""
    import random
    rnd = random.Random(21)
    failures = [f for f in (_random_lmhead_case(i, rnd, dev) for i in range(60)) if f is not None]
    assert not failures, failures
    # the smallest ragged tiles, alone in their group
    for tokens, vocab, hdim in [(1, 8, 64), (64, 16, 64), (2, 264, 128), (3, 24, 64), (3, 280, 64), (5, 2056, 64)]:
        g = torch.Generator(device=dev).manual_seed(vocab)
        h = torch.randn(tokens, hdim, generator=g, device=dev).to(torch.bfloat16)
        w = (torch.randn(vocab, hdim, generator=g, device=dev) * 0.2).to(torch.bfloat16)
        y = torch.randint(0, vocab, (tokens,), generator=g, device=dev)
        lp, ent, lse = mrl.lmhead_logprob(h, w, y)
        z = h.float() @ w.float().t()
        assert (lse - torch.logsumexp(z, -1)).abs().max().item() < 1e-4, (tokens, vocab, hdim)
        assert (lp - torch.log_softmax(z, -1).gather(-1, y[:, None])[:, 0]).abs().max().item() < 2e-4
        assert torch.isfinite(ent).all().item()


def _random_value_side_case(i, rnd, dev):
    """One random case of the KL-penalised rewards, the critic value loss, masked whitening and the
    group advantages against the oracle."""
    gen = torch.Generator().manual_seed(800 + i)
    batch = rnd.choice([1, 2, 7, 64, 257])
    width = rnd.choice([2, 3, 31, 257, 2048, 3000])
    old = -torch.rand(batch, width, generator=gen) * 5
    ref = old + torch.randn(batch, width, generator=gen) * 0.3
    lens = torch.randint(1, width + 1, (batch, 1), generator=gen)
    scores = torch.randn(batch, generator=gen)
    penalty = rnd.choice(["kl", "abs", "mse", "low_var_kl"])
    want, want_kl = o_adv.kl_token_level_rewards(old, ref, lens, scores, 0.05, penalty)
    got, got_kl = mrl.kl_token_level_rewards(old.to(dev), ref.to(dev), lens.to(dev), scores.to(dev), 0.05, penalty)
    # exp(c) - c - 1 cancels for small c: the mean KL carries an absolute error of a few fp32 ulps of 1
    if not ((got.cpu() - want).abs().max().item() < 1e-6 and abs(got_kl - want_kl) <= 1e-5 * abs(want_kl) + 2e-7):
        return (i, "kl_rewards", batch, width, penalty)
    # value loss
    values = torch.randn(batch, width, generator=gen)
    vp = values + torch.randn(batch, width, generator=gen) * 0.4
    returns = values + torch.randn(batch, width, generator=gen)
    vlens = torch.randint(0, width + 1, (batch, 1), generator=gen)
    vlens[0] = max(1, width // 2)
    mask = o_pack.generate_mask(vp, vlens).float()
    vo = vp.clone().requires_grad_()
    w_loss, w_frac = o_loss.value_loss(vo, returns, values, mask, 0.2)
    (g_o,) = torch.autograd.grad(w_loss, vo)
    vd = vp.to(dev).requires_grad_()
    g_loss, out = mrl.value_loss(vd, returns.to(dev), values.to(dev), cliprange_value=0.2, response_length=vlens.to(dev))
    (g,) = torch.autograd.grad(g_loss, vd)
    if not (abs(g_loss.item() - w_loss.item()) <= 1e-4 * abs(w_loss.item()) + 1e-8 and (g.cpu() - g_o).abs().max().item() < 1e-6
            and abs(out[2].item() - w_frac.item()) <= 1e-5 * abs(w_frac.item()) + 1e-8):
        return (i, "value_loss", batch, width, g_loss.item(), w_loss.item())
    # whitening / variance
    if int(mask.sum()) >= 2:
        for shift in (True, False):
            w = o_loss.masked_whiten(values, mask, shift_mean=shift)
            gw = mrl.masked_whiten(values.to(dev), mask.to(dev), shift_mean=shift)
            if not (gw.cpu() - w).abs().max().item() < 2e-5 * max(1.0, w.abs().max().item()):
                return (i, "whiten", batch, width, shift, (gw.cpu() - w).abs().max().item())
    # group advantages
    group = rnd.choice([2, 3, 8, 16])
    nb = group * rnd.randint(1, 6)
    L = rnd.choice([1, 5, 300])
    rewards = torch.randn(nb, 1, generator=gen) if rnd.random() < 0.5 else torch.bernoulli(torch.full((nb, 1), 0.5), generator=gen)
    alens = torch.randint(0, L + 1, (nb,), generator=gen)
    amask = o_pack.generate_mask(torch.zeros(nb, L), alens)
    wa, _ = o_adv.compute_group_norm_advantage_return(rewards, amask, torch.zeros(nb, 1), group)
    ga, _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), amask.to(dev), torch.zeros(nb, 1), group)
    if not (ga.cpu() - wa).abs().max().item() < 1e-6 * max(1.0, wa.abs().max().item()):
        return (i, "advantage", nb, group, L, (ga.cpu() - wa).abs().max().item())
    return None


def test_value_side_random_shapes(dev):
    """Randomised test of kl_token_level_rewards, value_loss (forward, clip fraction, gradient),
    masked_whiten and compute_group_norm_advantage_return against the oracle: batch 1..257, width
    2..3000, every KL estimator, empty rows, gaussian and 0/1 rewards."""
    import random
    rnd = random.Random(41)
    failures = [f for f in (_random_value_side_case(i, rnd, dev) for i in range(60)) if f is not None]
    assert not failures, failures


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_multimodal_logprob_computer(dev, dtype):
    """logprob_computer.py:40-70: the window's logits scored against `responses`; here without the
    [B, L, V] copy of the reference and with a gradient.  Oracle: the reference's own composition
    (truncate_middle_and_pad -> compute_log_probs; entropy over the full output)."""
    gen = torch.Generator().manual_seed(77)
    n_seq, seq_len, vocab, resp_w = 5, 23, 520, 9
    plen = torch.tensor([[1], [3], [5], [2], [20]], dtype=torch.int32)
    rlen = torch.tensor([[9], [4], [0], [7], [9]], dtype=torch.int32)       # the last window runs past seq_len
    out = (torch.randn(n_seq, seq_len, vocab, generator=gen) * 2).to(dtype)
    responses = torch.randint(0, vocab, (n_seq, resp_w), generator=gen)
    b = {"responses": responses, "prompt_length": plen, "response_length": rlen}
    window = o_pack.response_window(plen, rlen)
    zo = out.float().requires_grad_()
    want = o_vocab.compute_log_probs(o_pack.truncate_middle_and_pad(responses, zo, window), responses)
    want_h = o_vocab.vocab_parallel_entropy(out.float())
    g_out = torch.randn(n_seq, resp_w, generator=gen)
    (g_o,) = torch.autograd.grad(want, zo, g_out)
    comp = mrl.MultimodalLogProbComputer()
    zd = out.to(dev).requires_grad_()
    lp, ent = comp.compute(zd, _to_dev(b, dev), skip_entropy=False)
    assert lp.shape == (n_seq, resp_w) and ent.shape == (n_seq, seq_len)
    assert (lp.cpu() - want.detach()).abs().max().item() < TOL_LOGP
    assert (ent.detach().cpu() - want_h).abs().max().item() < TOL_LOGP
    # positions past a window hold exactly what the reference's zero padding gives
    assert lp[2].detach().cpu().tolist() == want[2].detach().tolist()
    (g,) = torch.autograd.grad(lp, zd, g_out.to(dev))
    assert g.dtype == dtype
    tol = 1e-5 if dtype == torch.float32 else 2 ** -8 * g_o.abs().max().item()
    assert (g.float().cpu() - g_o).abs().max().item() <= tol
    lp2, ent2 = comp.compute(out.to(dev), _to_dev(b, dev), skip_entropy=True)
    assert torch.equal(lp2, lp.detach()) and not ent2.any().item() and ent2.shape == lp2.shape


def test_loss_object_with_multimodal_computer(dev):
    """A loss object whose log-prob strategy was replaced does not take the fused sweep (which scores
    against `labels`): GRPO with the multimodal strategy equals the oracle's loss on the log-probs that
    strategy defines."""
    gen = torch.Generator().manual_seed(5)
    n_seq, seq_len, vocab, resp_w = 4, 19, 512, 8
    plen = torch.tensor([[2], [3], [1], [4]], dtype=torch.int32)
    rlen = torch.tensor([[8], [5], [8], [2]], dtype=torch.int32)
    out = torch.randn(n_seq, seq_len, vocab, generator=gen) * 2
    responses = torch.randint(0, vocab, (n_seq, resp_w), generator=gen)
    rmask = o_pack.generate_mask(responses, rlen)
    window = o_pack.response_window(plen, rlen)
    lp0 = o_vocab.compute_log_probs(o_pack.truncate_middle_and_pad(responses, out, window), responses)
    b = {"responses": responses, "prompt_length": plen, "response_length": rlen, "labels": torch.zeros(n_seq, seq_len, dtype=torch.int64),
         "advantages": torch.randn(n_seq, resp_w, generator=gen) * rmask,
         "old_log_prob": (lp0 + torch.randn(n_seq, resp_w, generator=gen) * 0.05) * rmask,
         "ref_log_prob": (lp0 + torch.randn(n_seq, resp_w, generator=gen) * 0.05) * rmask}
    zo = out.clone().requires_grad_()
    lp_o = o_vocab.compute_log_probs(o_pack.truncate_middle_and_pad(responses, zo, window), responses)
    want = o_loss.grpo_policy_loss(b["old_log_prob"], lp_o, b["ref_log_prob"], b["advantages"], torch.zeros_like(lp_o),
                                   rmask, 0.2, 0.01, "low_var_kl", 0.0)[0]
    (g_o,) = torch.autograd.grad(want, zo)
    f = mrl.GRPOActorLossFunc()
    f.logprob_computer = mrl.MultimodalLogProbComputer()
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.0})
    zd = out.to(dev).requires_grad_()
    got, _ = f.compute_loss(zd, _to_dev(b, dev))
    assert got.item() == pytest.approx(want.item(), rel=TOL_LOSS_REL)
    (g,) = torch.autograd.grad(got, zd)
    assert (g.cpu() - g_o).abs().max().item() < 1e-6


def test_injected_cross_entropy_reaches_the_loss_objects(dev):
    """set_vocab_parallel (the reference's hook, utils/compute.py:19-26): a caller's own cross entropy
    scores the rows of the loss objects too - forward-only log-probs and the training loss - and the
    fused sweep, which has its own scoring built in, steps aside."""
    gen = torch.Generator().manual_seed(12)
    logits, b, kw, _, _ = _make_batch(gen, 2, 3, 4, 12, 256, torch.float32, 2.0, 1)
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    calls = []

    def doubled_ce(vocab_parallel_logits, target):
        calls.append(tuple(vocab_parallel_logits.shape))
        return 2.0 * mrl.vocab_parallel_cross_entropy(vocab_parallel_logits, target)

    ref_fn = mrl.LossFuncFactory.get_instance("ray_grpo", "reference")
    plain = ref_fn.compute_loss(logits.to(dev), bd, forward_only=True, **kwd)
    f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.0})
    mrl.set_vocab_parallel(doubled_ce)
    try:
        got = ref_fn.compute_loss(logits.to(dev), bd, forward_only=True, **kwd)
        assert calls and torch.allclose(got, 2.0 * plain, atol=1e-6)
        n_calls = len(calls)
        zd = logits.to(dev).requires_grad_()
        loss, _ = f.compute_loss(zd, bd, **kwd)                     # would be the fused sweep by default
        assert len(calls) > n_calls
        (dz,) = torch.autograd.grad(loss, zd)
        assert torch.isfinite(dz).all().item() and dz.abs().max().item() > 0
    finally:
        mrl.set_vocab_parallel(None)
    zd = logits.to(dev).requires_grad_()
    loss_plain, _ = f.compute_loss(zd, bd, **kwd)
    assert abs(loss_plain.item() - loss.item()) > 1e-6             # the doubled scoring did change the loss


@pytest.mark.parametrize("layout", ["padded", "packed"])
def test_standard_computer_sweeps_only_window_rows(dev, layout):
    """The split path's log-prob strategy skips the logits rows that the response-window cut never
    reads (prompt rows, the last row, padding): same [B, L] values bit for bit as a sweep over every
    row, a gradient of exactly zero outside the windows and the same gradient inside, and rows
    outside the windows may hold anything (NaN here) without reaching the result."""
    from mindspeed_rl_amd.packing import preprocess_packed_seqs
    from mindspeed_rl_amd.vocab_ops import vocab_logprob_entropy
    gen = torch.Generator().manual_seed(123)
    n_seq, seq_len, vocab, resp_w = 6, 40, 777, 12
    plen = torch.tensor([[1], [7], [20], [3], [39], [28]], dtype=torch.int64)
    rlen = torch.tensor([[12], [5], [0], [12], [1], [12]], dtype=torch.int64)
    ids = torch.randint(0, vocab, (n_seq, seq_len), generator=gen)
    attn = (torch.arange(seq_len)[None, :] < (plen + rlen)).to(torch.int64)
    responses = torch.randint(0, vocab, (n_seq, resp_w), generator=gen)
    b = _to_dev({"responses": responses, "prompt_length": plen, "response_length": rlen,
                 "labels": torch.roll(ids, -1, 1)}, dev)
    kw = {}
    if layout == "packed":
        packed_ids, _, packed_labels, seqlens, cu = preprocess_packed_seqs(
            ids.to(dev), torch.roll(ids, -1, 1).to(dev), attn.to(dev), 1)
        b["labels"] = packed_labels
        n_rows = packed_ids.shape[1]
        kw = dict(use_remove_padding=True, seqlens_in_batch=seqlens, cu_seqlens_padded=cu, seq_len=resp_w)
        out = torch.randn(1, n_rows, vocab, generator=gen) * 2
    else:
        out = torch.randn(n_seq, seq_len, vocab, generator=gen) * 2
    comp = mrl.StandardLogProbComputer()
    active = comp._rows_in_windows(out.to(dev), b, kw).view(b["labels"].shape).bool()
    # the flags are the rows the cut reads: cutting a row-index tensor shows them
    idx = torch.arange(active.numel(), device=dev, dtype=torch.float32).view(active.shape) + 1
    if layout == "packed":
        picked = mrl.postprocess_packed_seqs(idx, seqlens, cu, resp_w, prompt_length=b["prompt_length"])
    else:
        picked = mrl.truncate_prompt_and_pad(responses.to(dev), idx, mrl.response_window(b["prompt_length"], b["response_length"]))
    want_active = torch.zeros(active.numel() + 1, dtype=torch.bool, device=dev)
    want_active[picked.long().flatten()] = True
    assert torch.equal(active.flatten(), want_active[1:])
    assert 0 < active.sum().item() < active.numel()

    zd = out.to(dev).requires_grad_()
    lp, ent = comp.compute(zd, b, skip_entropy=False, **kw)
    g_out = torch.randn(n_seq, resp_w, generator=gen).to(dev)
    (g,) = torch.autograd.grad((lp * g_out).sum() + 0.3 * ent.sum(), zd)
    # every row swept, then the same cut
    z2 = out.to(dev).requires_grad_()
    lp_all, ent_all, _ = vocab_logprob_entropy(z2, b["labels"])
    if layout == "packed":
        cut = lambda x: mrl.postprocess_packed_seqs(x, seqlens, cu, resp_w, prompt_length=b["prompt_length"])
    else:
        cut = lambda x: comp._get_log_probs_remove_prompt_pad(x, b)
    lp2, ent2 = cut(lp_all), cut(ent_all)
    (g2,) = torch.autograd.grad((lp2 * g_out).sum() + 0.3 * ent2.sum(), z2)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)
    assert torch.equal(g, g2)
    assert not g.view(-1, vocab)[~active.flatten()].any().item()
    # rows outside the windows are not read
    poisoned = out.to(dev).clone()
    poisoned.view(-1, vocab)[~active.flatten()] = float("nan")
    lp3, ent3 = comp.compute(poisoned, b, skip_entropy=False, **kw)
    assert torch.equal(lp3, lp.detach()) and torch.equal(ent3, ent.detach())


def test_fused_lmhead_policy_loss_skips_rows_without_response(dev):
    """With long prompts most rows carry no live response token: the chunked lm_head step gathers the
    live rows and runs its GEMMs on them alone.  Same loss, statistics, dHidden and dWeight as with
    every row projected (up to how a GEMM rounds when its row count changes), and dHidden exactly
    zero on the skipped rows.  A mask that switches off response tokens drops their rows as well."""
    gen = torch.Generator().manual_seed(31)
    vocab, hdim = 2048, 128
    _, b, kw, _, _ = _make_batch(gen, 2, 4, 3, 12, vocab, torch.bfloat16, 1.0, 2, prompt_hi=30)
    total = b["labels"].shape[1]
    n_seq, resp_w = b["advantages"].shape
    h = torch.randn(1, total, hdim, generator=gen).to(torch.bfloat16)
    w = (torch.randn(vocab, hdim, generator=gen) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    rmask = o_pack.generate_mask(torch.zeros(n_seq, resp_w), b["response_length"])
    mask = rmask * (torch.rand(n_seq, resp_w, generator=gen) > 0.3)
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    res = {}
    for compact in (True, False):
        hd, wd = h.to(dev).requires_grad_(), w.to(dev).requires_grad_()
        loss, out = mrl.fused_lmhead_policy_loss(hd, wd, bd, packed=True, seqlens=kwd["seqlens_in_batch"],
                                                 cu_seqlens=kwd["cu_seqlens_padded"], ref_log_prob=bd["ref_log_prob"],
                                                 mask=mask.to(dev), clip_low=0.2, clip_high=0.2, kl_penalty="low_var_kl",
                                                 kl_coef=0.01, entropy_coeff=0.002, chunk_rows=16, compact_rows=compact)
        dh, dw = torch.autograd.grad(loss, [hd, wd])
        res[compact] = (loss.item(), out.cpu(), dh.float().cpu()[0], dw.float().cpu())
    (l1, o1, dh1, dw1), (l0, o0, dh0, dw0) = res[True], res[False]
    assert l1 == pytest.approx(l0, rel=1e-5, abs=1e-8)
    assert torch.allclose(o1, o0, rtol=1e-5, atol=1e-7)
    assert (dh1 - dh0).abs().max().item() <= 2 ** -7 * dh0.abs().max().item()
    assert (dw1 - dw0).abs().max().item() <= 2 ** -7 * dw0.abs().max().item()
    # rows of the packed stream that hold a live token, from the oracle's own window cut
    idx = torch.arange(1, total + 1, dtype=torch.float32).view(1, total)
    picked = o_pack.postprocess_packed_seqs(idx, kw["seqlens_in_batch"], kw["cu_seqlens_padded"], resp_w,
                                            prompt_length=b["prompt_length"])
    live = torch.zeros(total + 1, dtype=torch.bool)
    live[(picked * mask).long().flatten()] = True
    live = live[1:]
    assert live.sum().item() * 20 <= total * 19            # the case does take the compacted path
    assert not dh1[~live].any().item()
    assert dh1[live].abs().sum(1).min().item() > 0


def test_lmhead_logprob_row_active(dev):
    """Only flagged rows are projected and scored; the others return zeros."""
    gen = torch.Generator().manual_seed(8)
    tokens, vocab, hdim = 301, 1000, 128
    h = torch.randn(tokens, hdim, generator=gen).to(torch.bfloat16).to(dev)
    w = (torch.randn(vocab, hdim, generator=gen) * (2.0 / hdim ** 0.5)).to(torch.bfloat16).to(dev)
    y = torch.randint(0, vocab, (tokens,), generator=gen).to(dev)
    act = (torch.rand(tokens, generator=gen) > 0.6).to(dev)
    full = mrl.lmhead_logprob(h, w, y)
    part = mrl.lmhead_logprob(h.view(1, tokens, hdim), w, y.view(1, tokens), row_active=act.view(1, tokens))
    for a, p in zip(full, part):
        assert p.shape == (1, tokens)
        assert not p.view(-1)[~act].any().item()
        assert (p.view(-1)[act] - a[act]).abs().max().item() < 2e-5
    none = mrl.lmhead_logprob(h, w, y, row_active=torch.zeros(tokens, dtype=torch.uint8, device=dev))
    assert all(not t.any().item() and t.shape == (tokens,) for t in none)
    with pytest.raises(ValueError):
        mrl.lmhead_logprob(h, w, y, row_active=act[:-1])


@pytest.mark.parametrize("fused", [True, False])
def test_loss_on_logits_that_are_views_or_products(dev, fused):
    """The logits a model hands over are the result of a projection, possibly a transposed or sliced
    view of it: loss and the gradients that reach hidden states and weight equal the oracle's, with
    and without the in-place gradient."""
    gen = torch.Generator().manual_seed(12)
    n_seq, seq_len, vocab, hdim = 4, 24, 1024, 64
    plen = torch.tensor([[3], [1], [5], [2]])
    rlen = torch.tensor([[10], [20], [7], [15]])
    resp_w = int(rlen.max())
    ids = torch.randint(0, vocab, (n_seq, seq_len), generator=gen)
    rmask = o_pack.generate_mask(torch.zeros(n_seq, resp_w), rlen)
    b = {"labels": torch.roll(ids, -1, 1), "responses": torch.zeros(n_seq, resp_w, dtype=torch.int64),
         "response_length": rlen, "prompt_length": plen,
         "advantages": torch.randn(n_seq, resp_w, generator=gen) * rmask,
         "old_log_prob": -torch.rand(n_seq, resp_w, generator=gen) * rmask * 3,
         "ref_log_prob": -torch.rand(n_seq, resp_w, generator=gen) * rmask * 3}
    meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.001)
    h = torch.randn(n_seq, seq_len, hdim, generator=gen)
    w = torch.randn(vocab, hdim, generator=gen) * 0.3
    projections = {
        "product": lambda hh, ww: hh @ ww.t(),
        "transposed view": lambda hh, ww: (hh.transpose(0, 1).contiguous() @ ww.t()).transpose(0, 1),
        "slice of a padded vocabulary": lambda hh, ww: (hh @ torch.cat([ww, torch.zeros(8, hdim, device=ww.device)]).t())[..., :vocab],
    }
    bd = _to_dev(b, dev)
    for name, project in projections.items():
        ho, wo = h.clone().requires_grad_(), w.clone().requires_grad_()
        want, _ = o_loss.grpo_compute_loss(project(ho, wo).contiguous(), b, meta)
        gh_o, gw_o = torch.autograd.grad(want, [ho, wo])
        for inplace in (False, True):
            f = mrl.GRPOActorLossFunc()
            f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                                  "entropy_coeff": 0.001})
            hd, wd = h.to(dev).requires_grad_(), w.to(dev).requires_grad_()
            got, _ = f.compute_loss(project(hd, wd), bd, fused=fused, grad_inplace=inplace)
            gh, gw = torch.autograd.grad(got, [hd, wd])
            assert got.item() == pytest.approx(want.item(), rel=TOL_LOSS_REL, abs=1e-7), name
            assert (gh.cpu() - gh_o).abs().max().item() < 1e-6, name
            assert (gw.cpu() - gw_o).abs().max().item() < 1e-6, name


@pytest.mark.parametrize("fused", [True, False])
def test_one_loss_object_over_interleaved_micro_batches(dev, fused):
    """A pipeline schedule runs the forward of several micro-batches of different shapes through ONE
    loss object and their backwards later, in another order: every loss and gradient equals the
    oracle's for its own micro-batch (nothing is shared between calls)."""
    micro_batch = _small_padded_micro_batch
    meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.001)
    items = [micro_batch(1, 4, 30, 512), micro_batch(2, 7, 19, 1032), micro_batch(3, 2, 40, 256)]
    want = []
    for z, b in items:
        zo = z.clone().requires_grad_()
        loss_o, _ = o_loss.grpo_compute_loss(zo, b, meta)
        (g_o,) = torch.autograd.grad(loss_o * 0.25, zo)
        want.append((loss_o.item(), g_o))
    for extra in ({}, {"grad_inplace": True}, {"expected_grad_scale": 0.25}):
        f = mrl.GRPOActorLossFunc()
        f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                              "entropy_coeff": 0.001})
        leaves, losses = [], []
        for z, b in items:
            zd = z.to(dev).requires_grad_()
            loss, _ = f.compute_loss(zd * 1.0, _to_dev(b, dev), fused=fused, **extra)     # a non-leaf: in-place is legal
            leaves.append(zd)
            losses.append(loss)
        for i in (1, 0, 2):
            (losses[i] * 0.25).backward()
        for i in range(3):
            assert losses[i].item() == pytest.approx(want[i][0], rel=TOL_LOSS_REL, abs=1e-7)
            assert (leaves[i].grad.cpu() - want[i][1]).abs().max().item() < 1e-6


def _pack_sequence_logits(seq_logits, seqlens, cu, total):
    """The stand-in for the model of the dynamic-batching test: row cu[i] + j of the packed
    [1, T, V] logits is what the model emits for position j of sequence i; alignment rows are 0."""
    out = torch.zeros(1, total, seq_logits.shape[-1], dtype=seq_logits.dtype, device=seq_logits.device)
    for i, n in enumerate(seqlens.tolist()):
        start = int(cu[i])
        out[0, start:start + n] = seq_logits[i, :n]
    return out


@pytest.mark.parametrize("algo", ["grpo", "dapo"])
def test_dynamic_micro_batches_end_to_end(dev, algo):
    """How the reference chunks an update when use_dynamic_bsz is on (utils/seqlen_balancing.py:339-380,
    models/base/base_training_engine.py:160-187, 238-270): 80 ragged sequences on the device are cut
    into token-budget micro-batches, each is packed, scored and back-propagated with loss / n_micro
    through ONE loss object with use_dynamic_bsz / actual_micro_batch_size.  The partitions, every
    micro-batch's loss and statistics, the summed loss and every sequence's dlogits equal the
    oracle's run over the oracle's own partitions, fused and split.  The DAPO variant applies the
    dynamic-sampling filter first (workers/dynamic_sampling.py:81-86): groups whose rewards are all
    equal never reach the loss."""
    from mindspeed_rl_amd import seqlen_balancing as bal
    from oracle import balancing as o_bal
    gen = torch.Generator().manual_seed(77 if algo == "grpo" else 78)
    n_prompts, group, vocab, align = 10, 8, 1032, 2
    n_all = n_prompts * group
    rlen = torch.randint(4, 61, (n_all, 1), generator=gen, dtype=torch.int32)
    plen = torch.randint(1, 7, (n_all, 1), generator=gen, dtype=torch.int32)
    width, resp_w = int((plen + rlen).max()), int(rlen.max())
    ids = torch.randint(0, vocab, (n_all, width), generator=gen)
    ids = ids * o_pack.generate_mask(ids, plen + rlen)
    seq_logits = torch.randn(n_all, width, vocab, generator=gen) * 2
    p = torch.rand(n_prompts, 1, generator=gen)
    p[1], p[4], p[7] = 0.0, 1.0, 0.0                       # three groups with all-equal rewards
    rewards = torch.bernoulli(p.repeat(1, group).reshape(n_all, 1), generator=gen)
    rmask = o_pack.generate_mask(torch.zeros(n_all, resp_w), rlen)
    adv, _ = o_adv.compute_group_norm_advantage_return(rewards, rmask, rlen, group)
    labels_pad = torch.cat([ids[:, 1:], torch.zeros(n_all, 1, dtype=ids.dtype)], 1)
    full = {"input_ids": ids, "responses": torch.zeros(n_all, resp_w, dtype=torch.int64), "response_length": rlen,
            "prompt_length": plen, "advantages": adv}
    lp0 = o_loss.logprob_computer(seq_logits, dict(full, labels=labels_pad), True)[0]
    full["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    full["ref_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    if algo == "dapo":
        keep_o = o_adv.dynamic_sampling_keep(rewards.flatten().numpy(), group)
        keep = mrl.dynamic_sampling_keep(rewards.flatten().to(dev), group)
        assert keep == keep_o and 0 < len(keep) <= n_all - 3 * group
        full = {k: v[keep] for k, v in full.items()}
        seq_logits = seq_logits[keep]
        meta_o = dict(clip_ratio=0.2, clip_higher_enable=True, clip_ratio_low=0.2, clip_ratio_high=0.28,
                      token_level_loss=True, entropy_coeff=0.001)
        meta_d = dict(meta_o)
        oracle_loss, make = o_loss.dapo_compute_loss, mrl.DAPOActorLossFunc
    else:
        meta_o = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.001)
        meta_d = {"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                  "entropy_coeff": 0.001}
        oracle_loss, make = o_loss.grpo_compute_loss, mrl.GRPOActorLossFunc
    n_seq = full["input_ids"].shape[0]
    max_tokens, max_bsz = 300, 12

    # ---- the oracle: its own partitions, CPU packing, CPU loss
    lengths = (full["prompt_length"] + full["response_length"]).flatten().tolist()
    parts_o = o_bal.rearrange_micro_batches(lengths, max_tokens, dynamic_max_batch_size=max_bsz)
    n_micro = len(parts_o)
    assert n_micro >= 5 and sorted(i for part in parts_o for i in part) == list(range(n_seq))
    want_grads, want_losses, want_stats = {}, [], []
    for part in parts_o:
        mb = {k: v[part] for k, v in full.items()}
        lab = torch.cat([mb["input_ids"][:, 1:], torch.zeros(len(part), 1, dtype=ids.dtype)], 1)
        mask1d = o_pack.generate_mask(mb["input_ids"], mb["prompt_length"] + mb["response_length"])
        _, _, p_lab, seqlens, cu = o_pack.preprocess_packed_seqs(mb["input_ids"], lab, mask1d, align)
        z = _pack_sequence_logits(seq_logits[part], seqlens, cu, p_lab.shape[1]).requires_grad_()
        mb["labels"] = p_lab
        loss, stats = oracle_loss(z, mb, meta_o, use_remove_padding=True, seqlens_in_batch=seqlens,
                                  cu_seqlens_padded=cu, seq_len=width, use_dynamic_bsz=True,
                                  actual_micro_batch_size=n_seq / n_micro)
        (loss / n_micro).backward()
        want_losses.append(loss.item())
        want_stats.append(stats)
        for i, s in enumerate(part):
            want_grads[s] = z.grad[0, int(cu[i]):int(cu[i]) + int(seqlens[i])].clone()

    # ---- the device path: split on the device batch, pack with the index-map kernels, one loss object
    full_d = _to_dev(full, dev)
    logits_d = seq_logits.to(dev)
    for fused in (True, False):
        f = make()
        f.add_loss_meta_info(meta_d)
        batches, parts = bal.split_batches_with_dynamic_bsz(full_d, max_tokens, max_bsz)
        assert parts == parts_o
        total_loss = 0.0
        for k, (mb, part) in enumerate(zip(batches, parts)):
            lab = torch.cat([mb["input_ids"][:, 1:], torch.zeros(len(part), 1, dtype=ids.dtype, device=dev)], 1)
            mask1d = mrl.generate_mask(mb["input_ids"], mb["prompt_length"] + mb["response_length"])
            _, _, p_lab, seqlens, cu = mrl.preprocess_packed_seqs(mb["input_ids"], lab, mask1d, align)
            zd = _pack_sequence_logits(logits_d[part], seqlens.cpu(), cu.cpu(), p_lab.shape[1]).requires_grad_()
            mb["labels"] = p_lab
            loss, stats = f.compute_loss(zd, mb, fused=fused, use_remove_padding=True, seqlens_in_batch=seqlens,
                                         cu_seqlens_padded=cu, seq_len=width, use_dynamic_bsz=True,
                                         actual_micro_batch_size=n_seq / n_micro, index=None)
            (loss / n_micro).backward()
            assert loss.item() == pytest.approx(want_losses[k], rel=TOL_LOSS_REL, abs=1e-7)
            for name, v in want_stats[k].items():
                assert stats[name] == pytest.approx(v, rel=TOL_LOSS_REL, abs=1e-6), (k, name)
            total_loss += loss.item() / n_micro
            cu_h, len_h = cu.cpu(), seqlens.cpu()
            for i, s in enumerate(part):
                got = zd.grad[0, int(cu_h[i]):int(cu_h[i]) + int(len_h[i])].cpu()
                assert (got - want_grads[s]).abs().max().item() < 1e-6, (k, s)
            if align > 1 and int(cu_h[-1]) > int(len_h.sum()):
                pad_rows = torch.ones(int(cu_h[-1]), dtype=torch.bool)
                for i in range(len(part)):
                    pad_rows[int(cu_h[i]):int(cu_h[i]) + int(len_h[i])] = False
                assert not zd.grad[0][pad_rows.to(dev)].any().item()      # alignment rows get no gradient
        assert total_loss == pytest.approx(sum(want_losses) / n_micro, rel=TOL_LOSS_REL, abs=1e-7)
        if fused:
            # upstream 1/n_micro is learned from the first backward: one rescale pass, not n_micro
            assert f.grad_scale_state(dev).rescales.item() == 1


def test_config4_whole_batch_in_micro_batches(dev):
    """configs[4] whole, as `bench.py --workload c4` runs it: 8 x 16 responses of 8 k - 32 k tokens, the
    dynamic-sampling filter first, the kept sequences cut into micro-batches of at most 65 536 tokens by the
    Karmarkar-Karp partitioner (the oracle's partitions must be the same), every micro-batch's logits
    ([T <= 65 536, 129 280] bf16, up to 17 GB) generated on the device, ONE DAPO loss object with
    use_dynamic_bsz / actual_micro_batch_size, (loss / n_micro).backward().  The oracle cannot follow at
    this size, so every micro-batch is held to the size-independent properties: the fused sweep and the
    split kernels (independent code) agree on loss, statistics and every dlogit; every dlogits row sums to
    zero; rows without a response token are exactly zero; sampled rows match the oracle's log-prob and
    entropy and lie in the span of the two gradient directions the closed form allows.  The upstream
    gradient 1 / n_micro is learned once: one rescale pass in the whole batch."""
    import bench
    import gc
    from mindspeed_rl_amd import seqlen_balancing as bal
    from oracle import balancing as o_bal
    gc.collect()
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 80 * 2 ** 30:
        pytest.skip("needs more free HBM")
    full, keep, n_all = bench.make_c4_batch(torch, mrl, dev, 0)
    group, vocab = bench.C4["group"], bench.C4["vocab"]
    n_seq = len(keep)
    assert n_all == 128 and n_seq % group == 0 and 3 * group <= n_seq < n_all
    kept_groups = sorted(set(i // group for i in keep))
    assert keep == [g * group + j for g in kept_groups for j in range(group)]
    # every kept group mixes rewards, so its advantages have both signs; lengths are in range
    adv0 = full["advantages"][:, 0].view(-1, group)
    assert (adv0.max(1).values > 0).all().item() and (adv0.min(1).values < 0).all().item()
    rl = full["response_length"].flatten()
    assert rl.min().item() >= 8192 and rl.max().item() <= 32768
    batches, parts = bal.split_batches_with_dynamic_bsz(full, 65536, None)
    lengths = (full["prompt_length"] + full["response_length"]).flatten().tolist()
    assert parts == o_bal.rearrange_micro_batches(lengths, 65536, dynamic_max_batch_size=None)
    n_micro = len(parts)
    assert sorted(i for part in parts for i in part) == list(range(n_seq))
    assert n_micro >= (sum(lengths) + 65535) // 65536 and all(sum(lengths[i] for i in part) <= 65536 for part in parts)
    f = mrl.LossFuncFactory.get_instance("ray_dapo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "clip_higher_enable": True, "clip_ratio_low": 0.2,
                          "clip_ratio_high": 0.28, "token_level_loss": True, "entropy_coeff": 0.001})
    ref_fn = mrl.LossFuncFactory.get_instance("ray_grpo", "reference")
    gen = torch.Generator(device=dev).manual_seed(0)
    cpu_gen = torch.Generator().manual_seed(4)
    total_loss, rows_seen, checked = 0.0, 0, 0
    for k, (mb, part) in enumerate(zip(batches, parts)):
        mb = dict(mb)
        logits, kw, total = bench.c4_micro_batch_inputs(torch, mrl, mb, dev, gen, ref_fn)
        rows_seen += total
        flat, flat_labels = logits.view(-1, vocab), mb["labels"].reshape(-1)
        cu = kw["cu_seqlens_padded"].cpu().tolist()
        live = torch.zeros(total, dtype=torch.bool)
        for i, r in enumerate(mb["response_length"].flatten().tolist()):
            live[cu[i]:cu[i] + r] = True                     # 1-token prompts: the first R_i rows of a sequence
        live_d = live.to(dev)
        live_idx = torch.nonzero(live).flatten()
        pick = torch.cat([live_idx[torch.randint(0, live_idx.numel(), (6,), generator=cpu_gen)],
                          torch.nonzero(~live).flatten()[:2]])
        pick_d = pick.to(dev)
        zs, ys = flat[pick_d].float().cpu(), flat_labels[pick_d].cpu()
        z1 = logits.detach().requires_grad_()
        dyn = dict(use_dynamic_bsz=True, actual_micro_batch_size=n_seq / n_micro, index=None)
        loss_f, stats_f = f.compute_loss(z1, mb, fused=True, **dyn, **kw)
        (loss_f / n_micro).backward()
        dz_f = z1.grad.view(-1, vocab)
        total_loss += loss_f.item() / n_micro
        got = dz_f[pick_d].float().cpu() * n_micro
        # the split kernels on the same micro-batch, gradient written over the logits
        z2 = logits.detach().requires_grad_()
        loss_s, stats_s = f.compute_loss(z2, mb, fused=False, grad_inplace=True, **dyn, **kw)
        (dz_s,) = torch.autograd.grad(loss_s / n_micro, z2)
        dz_s = dz_s.view(-1, vocab)
        assert loss_s.item() == pytest.approx(loss_f.item(), rel=TOL_LOSS_REL), k
        for name in stats_f:
            assert stats_s[name] == pytest.approx(stats_f[name], rel=TOL_LOSS_REL, abs=2e-6), (k, name)
        scale, worst_sum, worst_diff = 0.0, 0.0, 0.0
        for lo in range(0, total, 8192):
            a, c = dz_f[lo:lo + 8192].float(), dz_s[lo:lo + 8192].float()
            scale = max(scale, a.abs().max().item())
            worst_diff = max(worst_diff, (a - c).abs().max().item())
            worst_sum = max(worst_sum, a.sum(-1).abs().max().item())
            dead = ~live_d[lo:lo + 8192]
            if dead.any().item():
                assert a.abs().amax(-1)[dead].max().item() == 0 and c.abs().amax(-1)[dead].max().item() == 0, k
            del a, c
        assert scale > 0 and worst_diff <= 2 ** -7 * scale and worst_sum <= 0.02 * scale, k
        # sampled rows: the gradient is c0 (onehot - p) - c1 p (z - E z) for some c0, c1
        p = torch.softmax(zs, -1)
        onehot = torch.zeros_like(p)
        onehot[torch.arange(len(ys)), ys] = 1.0
        basis0, basis1 = onehot - p, -(p * (zs - (p * zs).sum(-1, keepdim=True)))
        for i in range(len(pick)):
            if not live[pick[i]]:
                assert not got[i].any().item()
                continue
            a = torch.stack([basis0[i], basis1[i]], 1).double()
            coef = torch.linalg.lstsq(a, got[i].double().unsqueeze(1)).solution
            resid = (a @ coef).squeeze(1) - got[i].double()
            assert resid.abs().max().item() <= 2 ** -8 * got[i].abs().max().item() + 1e-12, (k, i)
            checked += 1
        del z1, z2, dz_f, dz_s, logits, flat
    assert rows_seen == sum(lengths) and checked >= 5 * n_micro
    assert total_loss == total_loss and abs(total_loss) < 10           # finite
    assert f.grad_scale_state(dev).rescales.item() == 1


def _small_padded_micro_batch(seed, n_seq, seq_len, vocab):
    g = torch.Generator().manual_seed(seed)
    plen = torch.randint(1, 5, (n_seq, 1), generator=g)
    rlen = torch.randint(1, seq_len - 5, (n_seq, 1), generator=g)
    resp_w = int(rlen.max())
    ids = torch.randint(0, vocab, (n_seq, seq_len), generator=g)
    rmask = o_pack.generate_mask(torch.zeros(n_seq, resp_w), rlen)
    b = {"labels": torch.roll(ids, -1, 1), "responses": torch.zeros(n_seq, resp_w, dtype=torch.int64),
         "response_length": rlen, "prompt_length": plen,
         "advantages": torch.randn(n_seq, resp_w, generator=g) * rmask,
         "old_log_prob": -torch.rand(n_seq, resp_w, generator=g) * rmask * 3,
         "ref_log_prob": -torch.rand(n_seq, resp_w, generator=g) * rmask * 3}
    return torch.randn(n_seq, seq_len, vocab, generator=g) * 2, b


def test_upstream_scale_is_learned_across_micro_batches(dev):
    """What the reference's caller does (models/base/base_training_engine.py:238-270): one loss object,
    n micro-batches, and the schedule back-propagates loss / n without telling the loss function.
    The fused sweep writes its gradients with the scale of the previous backward, so only the first
    micro-batch pays a rescale pass; every gradient equals the oracle's.  A change of the scale (a
    new number of micro-batches, a new loss scale) costs one more rescale, never a wrong gradient."""
    meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.001)
    f = mrl.GRPOActorLossFunc()
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.001})
    state = f.grad_scale_state(dev)
    assert state is f.grad_scale_state(dev) and state.learned.item() == 1.0 and state.rescales.item() == 0
    plan = [(0.25, 4), (0.5, 2), (1.0 / 3.0, 3)]                # (upstream, micro-batches); 1/3 is not a power of two
    expected_rescales, seed = 0, 100
    for upstream, n_micro in plan:
        expected_rescales += 1
        for _ in range(n_micro):
            seed += 1
            z, b = _small_padded_micro_batch(seed, 3 + seed % 3, 24, 520)
            zo = z.clone().requires_grad_()
            loss_o, _ = o_loss.grpo_compute_loss(zo, b, meta)
            (g_o,) = torch.autograd.grad(loss_o * upstream, zo)
            zd = z.to(dev).requires_grad_()
            loss, _ = f.compute_loss(zd, _to_dev(b, dev), fused=True)
            (loss * upstream).backward()
            assert loss.item() == pytest.approx(loss_o.item(), rel=TOL_LOSS_REL, abs=1e-7)
            assert (zd.grad.cpu() - g_o).abs().max().item() < 1e-6
            assert state.rescales.item() == expected_rescales
            assert state.learned.item() == torch.tensor(upstream, dtype=torch.float32).item()
    # an upstream gradient that cannot be a scale (0, inf, NaN) is honoured but not learned
    z, b = _small_padded_micro_batch(7, 3, 24, 520)
    zd = z.to(dev).requires_grad_()
    loss, _ = f.compute_loss(zd, _to_dev(b, dev), fused=True)
    (loss * 0.0).backward()
    assert not zd.grad.any().item() and state.learned.item() == torch.tensor(1.0 / 3.0).item()
    # an explicit expected_grad_scale bypasses the learned one
    zd = z.to(dev).requires_grad_()
    before = state.rescales.item()
    loss, _ = f.compute_loss(zd, _to_dev(b, dev), fused=True, expected_grad_scale=0.125)
    (loss * 0.125).backward()
    assert state.rescales.item() == before
    zo = z.clone().requires_grad_()
    (g_o,) = torch.autograd.grad(o_loss.grpo_compute_loss(zo, b, meta)[0] * 0.125, zo)
    assert (zd.grad.cpu() - g_o).abs().max().item() < 1e-6


@pytest.mark.parametrize("kind", ["logits", "lmhead"])
def test_two_backwards_over_one_retained_graph(dev, kind):
    """retain_graph=True: the second backward must not multiply the stored gradient by its upstream
    ratio a second time, and must leave the tensor the first backward handed out untouched."""
    meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.001)
    z, b = _small_padded_micro_batch(11, 4, 24, 520)
    bd = _to_dev(b, dev)
    if kind == "logits":
        # the oracle's cross entropy works in place like Megatron's and cannot be back-propagated twice:
        # one fresh graph per upstream value
        want = []
        for u in (0.5, 0.3, 0.5):
            zo = z.clone().requires_grad_()
            want.append(torch.autograd.grad(o_loss.grpo_compute_loss(zo, b, meta)[0] * u, zo))
        f = mrl.GRPOActorLossFunc()
        f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                              "entropy_coeff": 0.001})
        leaves = (z.to(dev).requires_grad_(),)
        loss, _ = f.compute_loss(leaves[0], bd, fused=True)
        tol = 1e-6
    else:
        g = torch.Generator().manual_seed(5)
        hdim = 64
        h = torch.randn(z.shape[0], z.shape[1], hdim, generator=g).to(torch.bfloat16)
        w = (torch.randn(520, hdim, generator=g) * 0.3).to(torch.bfloat16)
        want = []
        for u in (0.5, 0.3, 0.5):
            ho, wo = h.float().requires_grad_(), w.float().requires_grad_()
            loss_o, _ = o_loss.grpo_compute_loss(torch.nn.functional.linear(ho, wo).to(torch.bfloat16).float(), b, meta)
            want.append(torch.autograd.grad(loss_o * u, [ho, wo]))
        leaves = (h.to(dev).requires_grad_(), w.to(dev).requires_grad_())
        loss, _ = mrl.fused_lmhead_policy_loss(leaves[0], leaves[1], bd, packed=False, ref_log_prob=bd["ref_log_prob"],
                                               clip_low=0.2, clip_high=0.2, kl_penalty="low_var_kl", kl_coef=0.01,
                                               entropy_coeff=0.001)
        tol = None
    got = []
    for i, u in enumerate((0.5, 0.3, 0.5)):
        got.append(torch.autograd.grad(loss * u, leaves, retain_graph=(i < 2)))
    torch.cuda.synchronize()
    for grads, refs in zip(got, want):
        for a, r in zip(grads, refs):
            bound = tol if tol is not None else 2e-2 * r.abs().max().item()
            assert (a.float().cpu() - r).abs().max().item() <= bound
    # the first and the third backward had the same upstream value: identical results, separate storage
    for a, c in zip(got[0], got[2]):
        assert a.data_ptr() != c.data_ptr() and torch.equal(a, c)


def test_deferred_statistics_equal_the_eager_ones(dev):
    """deferred_stats=True takes the device-to-host copy of the statistics off the path between forward
    and backward: the floats that come out when the dict is finally read are those of the eager call,
    for every loss object, fused and split, and many deferred dicts may be outstanding at once."""
    gen = torch.Generator().manual_seed(3)
    logits, b, kw, _, _ = _make_batch(gen, 2, 4, 5, 30, 2048, torch.bfloat16, 2.0, 1)
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)
    metas = {("ray_grpo", "actor"): {"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                                     "entropy_coeff": 0.001},
             ("ray_dapo", "actor"): {"clip_ratio": 0.2, "clip_higher_enable": True, "clip_ratio_low": 0.2,
                                     "clip_ratio_high": 0.28, "token_level_loss": True, "entropy_coeff": 0.001},
             ("ray_ppo", "actor"): {"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.0), "entropy_coeff": 0.001}}
    held = []
    for key, meta in metas.items():
        for fused in (True, False):
            f = mrl.LossFuncFactory.get_instance(*key)
            f.add_loss_meta_info(meta)
            z = logits.to(dev).requires_grad_()
            loss_e, eager = f.compute_loss(z, bd, fused=fused, **kwd)
            loss_d, lazy = f.compute_loss(z, bd, fused=fused, deferred_stats=True, **kwd)
            (g,) = torch.autograd.grad(loss_d, z)                       # the backward runs before anyone looks
            assert type(eager) is dict and isinstance(lazy, mrl.DeferredStats) and set(lazy) == set(eager)
            held.append((eager, lazy, loss_e.item(), loss_d.item()))
    for eager, lazy, le, ld in held:
        assert le == ld and dict(lazy) == eager and all(isinstance(v, float) for v in lazy.values())
    # more outstanding dicts than pinned slots: the oldest are fetched when their slot comes round again
    f = mrl.GRPOActorLossFunc()
    f.add_loss_meta_info(metas[("ray_grpo", "actor")])
    z = logits.to(dev).requires_grad_()
    _, want = f.compute_loss(z, bd, fused=True, **kwd)
    many = [f.compute_loss(z, bd, fused=True, deferred_stats=True, **kwd)[1] for _ in range(300)]
    assert all(dict(m) == want for m in many)


@pytest.mark.parametrize("source", ["logits", "padded_logits_dapo_quarter", "hidden_states"])
def test_whole_step_captured_in_a_graph_and_replayed(dev, source):
    """compute_loss + backward captured once (torch.cuda.graph) and replayed on new inputs written into the
    same buffers: nothing on the path waits for the device or allocates outside torch's pool, the cleared
    words are cleared by a kernel, and the statistics stay on the device until they are read.  Every replay
    is checked against an eager step on the same inputs (bit-identical: the same kernels on the same data),
    with that eager work and synchronisations between the replays.  From the hidden states the live rows are
    not gathered (lm_head_compact_rows=False): their number would have to be read back."""
    gen = torch.Generator().manual_seed(77)
    f = mrl.GRPOActorLossFunc()
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.001})
    divide = 1.0                    # the schedule back-propagates loss / divide (number of micro-batches)
    if source == "padded_logits_dapo_quarter":
        # padded [B, S, V] fp32 logits, DAPO with a sequence-mean loss, and loss / 4 back-propagated: the
        # scale reaches the stored gradients through a device scalar, so it is part of the replay as well
        f = mrl.DAPOActorLossFunc()
        f.add_loss_meta_info({"clip_ratio": 0.2, "clip_higher_enable": True, "clip_ratio_low": 0.2,
                              "clip_ratio_high": 0.28, "token_level_loss": False, "entropy_coeff": 0.001})
        z0, b = _small_padded_micro_batch(5, 6, 24, 1032)
        kw, extra, divide = {}, {"fused": True}, 4.0
        fresh = lambda: [(torch.randn(z0.shape, generator=gen) * 2).to(dev)]
    elif source == "logits":
        logits, b, kw, _, _ = _make_batch(gen, 2, 4, 5, 30, 2048, torch.bfloat16, 2.0, 1)
        shapes, extra = [tuple(logits.shape)], {"fused": True}
        fresh = lambda: [(torch.randn(shapes[0], generator=gen) * 2).to(torch.bfloat16).to(dev)]
    else:
        vocab, hdim = 2048, 128
        _, b, kw, _, _ = _make_batch(gen, 2, 4, 5, 24, vocab, torch.bfloat16, 1.0, 2, prompt_hi=6)
        total = b["labels"].shape[1]
        extra = {"lm_head_compact_rows": False}
        fresh = lambda: [torch.randn(1, total, hdim, generator=gen).to(torch.bfloat16).to(dev),
                         (torch.randn(vocab, hdim, generator=gen) * (3.0 / hdim ** 0.5)).to(torch.bfloat16).to(dev)]
    bd, kwd = _to_dev(b, dev), _to_dev(kw, dev)

    def step(inputs):
        if source == "hidden_states":
            loss, stats = f.compute_loss(inputs[0], bd, lm_head_weight=inputs[1], **extra, **kwd)
        else:
            loss, stats = f.compute_loss(inputs[0], bd, **extra, **kwd)
        return loss, stats, torch.autograd.grad(loss / divide, inputs)

    static = [t.requires_grad_() for t in fresh()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):                       # warm-up off the default stream, as capture asks for
        for _ in range(2):
            step(static)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loss_g, stats_g, grads_g = step(static)
    torch.cuda.synchronize()
    assert isinstance(stats_g, mrl.DeferredStats)
    seen = set()
    for _ in range(4):
        new = fresh()
        with torch.no_grad():
            for dst, src in zip(static, new):
                dst.copy_(src)
        loss_e, stats_e, grads_e = step([t.clone().requires_grad_() for t in new])      # eager, between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert loss_g.item() == loss_e.item() and dict(stats_g) == stats_e
        for got, want in zip(grads_g, grads_e):
            assert torch.equal(got, want)
        seen.add(loss_e.item())
    assert len(seen) == 4                               # the replays did see different inputs


@pytest.mark.parametrize("upstream", [0.0, float("inf")])
def test_backward_with_a_zero_or_infinite_upstream_gradient(dev, upstream):
    """A skipped or overflowed loss-scale step reaches the loss as an upstream gradient of 0 or Inf.  It
    is applied like any other value (zeros, or infinities and NaN, come out - autograd's own product),
    it is NOT taken as the scale of the next sweep, and the next step is exact again.  What cannot be
    had afterwards is a second backward over the SAME retained graph: the stored gradients have been
    multiplied by 0 or Inf, so it yields NaN - a value that cannot pass for a gradient - rather than a
    wrong finite one."""
    meta = dict(clip_ratio=0.2, kl_coef=0.01, kl_penalty="low_var_kl", entropy_coeff=0.001)
    z, b = _small_padded_micro_batch(13, 4, 24, 520)
    bd = _to_dev(b, dev)
    zo = z.clone().requires_grad_()
    (want,) = torch.autograd.grad(o_loss.grpo_compute_loss(zo, b, meta)[0] * 0.5, zo)
    f = mrl.GRPOActorLossFunc()
    f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.01), "kl_penalty": "low_var_kl",
                          "entropy_coeff": 0.001})
    state = f.grad_scale_state(dev)
    zd = z.to(dev).requires_grad_()
    (g0,) = torch.autograd.grad(f.compute_loss(zd, bd, fused=True)[0] * 0.5, zd)          # learns 0.5
    assert state.learned.item() == 0.5
    loss, _ = f.compute_loss(zd, bd, fused=True)
    (g1,) = torch.autograd.grad(loss * upstream, zd, retain_graph=True)
    live = want != 0
    if upstream == 0.0:
        assert not g1.any().item()
    else:
        assert not torch.isfinite(g1.cpu()[live]).any().item()
    assert state.learned.item() == 0.5                               # not learned
    (g2,) = torch.autograd.grad(loss * 0.5, zd)                      # same graph again: cannot be recovered
    assert torch.isnan(g2.cpu()[live]).all().item()
    (g3,) = torch.autograd.grad(f.compute_loss(zd, bd, fused=True)[0] * 0.5, zd)          # the next step
    assert (g3.cpu() - want).abs().max().item() <= 1e-6 and torch.equal(g3, g0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bounds", [(0, 2048, 4096), (0, 1024, 2048, 3072, 4096), (0, 520, 528, 3000, 4096)])
def test_vocabulary_shards_merge_to_the_full_sweep(dev, dtype, bounds):
    """One tensor-parallel rank's share of the path, run for every rank in turn on one GPU: the
    per-shard statistics (12 bytes per token) merge to the oracle's full-vocabulary log-prob and
    entropy, and the shards' gradients, computed from the merged statistics, are the slices of the
    oracle's gradient.  Labels outside the vocabulary, a skipped row and temperature included."""
    gen = torch.Generator().manual_seed(len(bounds))
    rows, vocab, inv_t = 37, bounds[-1], 1.0 / 0.8
    z = _logits(gen, rows, vocab, dtype)
    y = torch.randint(0, vocab, (rows,), generator=gen)
    y[3], y[4] = bounds[1] - 1, bounds[1]                  # either side of a shard boundary
    active = torch.ones(rows, dtype=torch.uint8)
    active[5] = 0
    zo = (z.float() * inv_t).requires_grad_()
    lp_o = o_vocab.compute_log_probs(zo, y)
    h_o = o_vocab.vocab_parallel_entropy(zo)
    g_lp, g_h = torch.randn(rows, generator=gen), torch.randn(rows, generator=gen) * 0.1
    g_lp[5] = g_h[5] = 0.0
    (dz_o,) = torch.autograd.grad((lp_o * g_lp).sum() + (h_o * g_h).sum(), zo)
    dz_o = dz_o * inv_t
    zd, yd = z.to(dev), y.to(dev)
    shards = [zd[:, a:b] for a, b in zip(bounds[:-1], bounds[1:])]          # strided views, as a rank's slice
    stats = torch.stack([mrl.vocab_shard_stats(s, yd, a, inv_temperature=inv_t, row_active=active.to(dev))
                         for s, a in zip(shards, bounds[:-1])])
    assert stats.shape == (len(shards), rows, 3)
    lp, ent, lse = mrl.merge_vocab_shard_stats(stats)
    live = active.bool()
    assert (lp.cpu() - lp_o.detach())[live].abs().max().item() < TOL_LOGP
    assert (ent.cpu() - h_o.detach())[live].abs().max().item() < TOL_LOGP
    assert lp[5].item() == 0 and ent[5].item() == 0 and lse[5].item() == 0
    full_lp, full_ent, full_lse = mrl.vocab_logprob_entropy(zd, yd, inv_temperature=inv_t)
    assert (lp - full_lp)[live.to(dev)].abs().max().item() < 2e-5
    assert (ent - full_ent)[live.to(dev)].abs().max().item() < 2e-5
    dz = torch.cat([mrl.vocab_shard_backward(s, yd, a, lse, ent, g_lp.to(dev), g_h.to(dev), inv_temperature=inv_t)
                    for s, a in zip(shards, bounds[:-1])], dim=1)
    assert dz.dtype == dtype and dz.shape == (rows, vocab)
    tol = 1e-5 if dtype == torch.float32 else 2 ** -8 * dz_o.abs().max().item()
    assert (dz.float().cpu() - dz_o).abs().max().item() <= tol
    assert not dz[5].any().item()
    # a label outside every shard: the oracle (Megatron's target mask) scores the row maximum there,
    # a sharded run scores 0 - documented difference, no rank owns such a label
