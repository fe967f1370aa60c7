#!/usr/bin/env python3
"""Benchmark of the actor log-prob + GRPO loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c0|c2|c4|c4chunk|c3|c3fwd]

One step = one pass of the path over one synthetic packed batch resident in HBM: the fused
vocabulary sweep (log-prob + entropy + logsumexp), the unpack to [B, L], the fused policy loss
with its five statistics (one device-to-host copy), and the backward down to dlogits.  The
headline workload is the Qwen2.5-7B-shaped GRPO actor step: 16 prompts x 8 responses, response lengths
uniform in [512, 2048] (about 164k packed rows), vocabulary 152064, bf16 logits ~N(0, 3), labels
drawn from softmax(logits), clip 0.2, k3 KL 0.001, token-mean loss.

Prints ONE JSON line: tokens/s for the whole step, the roofline of the dominant kernel (the
sweep) from HIP events recorded on the launch stream inside the timed region, and a CPU
baseline: the oracle's restatement of the reference's torch op chain, timed on this host's cores
on a bounded row sample of the same workload.  Without --workload (or with --workload all) the
same line carries, under "other_workloads", a few steps of every other configuration: the
CPU-sized batch (c0), the padded layout (c2), the whole long-response DAPO batch in token-budget
micro-batches (c4), fp32 logits, an upstream gradient the loss object is not told (upstream0.25)
and the lm_head forward and training step (c3fwd, c3); the headline keys stay those of the
headline workload.  That run also measures roofline.traffic itself: two short child runs of this
script under rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), scaled by the copy probe of the same run.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "mindspeed-rl_amd"))

HBM_PEAK_GBPS = 8000.0

WORKLOADS = {
    # name: prompts, group, r_lo, r_hi, vocab, dtype, sigma, description
    "c1": dict(prompts=16, group=8, r_lo=512, r_hi=2048, vocab=152064, dtype="bf16", sigma=3.0,
               desc="configs[1]: Qwen2.5-7B-shaped GRPO actor step, 16x8 responses, R~U[512,2048], V=152064 bf16"),
    "c2": dict(prompts=16, group=8, r_lo=512, r_hi=2048, vocab=152064, dtype="bf16", sigma=3.0, layout="padded",
               empty_group=5, equal_group=3,
               desc="configs[2]: the configs[1] batch as padded [B,S,V] logits (S = longest sequence), one group of "
                    "empty responses and one group of all-equal rewards"),
    "c0": dict(prompts=4, group=4, r_lo=64, r_hi=256, vocab=32000, dtype="f32", sigma=2.0,
               desc="configs[0]: 4x4 responses, R~U[64,256], V=32000 fp32"),
    "c4chunk": dict(prompts=1, group=4, r_lo=8192, r_hi=24576, vocab=129280, dtype="bf16", sigma=3.0, loss="dapo",
                    desc="one ~64k-row chunk of configs[4]: 4 of a kept group's 16 responses, R~U[8192,24576], "
                         "V=129280 bf16, DAPO clip-higher 0.2/0.28, no KL, token-level loss"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="all", choices=["all"] + sorted(WORKLOADS) + ["c4", "c3fwd", "c3"],
                    help="all: the headline (c1) plus a few steps of every other workload under 'other_workloads'; "
                         "c4: configs[4] whole - 8x16 long responses, dynamic-sampling filter, 64k-token micro-batches; "
                         "c3fwd: the fused lm_head + log-prob forward of configs[3] (bf16 MFMA, logits never stored); "
                         "c3: configs[3] forward + backward from the hidden states (per chunk: logits product -> fused sweep -> dHidden and dW products)")
    ap.add_argument("--token-budget", type=int, default=65536,
                    help="c4 only: token budget of a micro-batch (configs[4]: 64k-token chunks)")
    ap.add_argument("--other-steps", type=int, default=3, help="steps of each entry of other_workloads")
    ap.add_argument("--tokens", type=int, default=163840, help="rows of the c3fwd workload")
    ap.add_argument("--entropy-coeff", type=float, default=0.001,
                    help="non-zero so that the forward computes entropy and the backward its gradient")
    ap.add_argument("--chunk-rows", type=int, default=32768,
                    help="c3 only: logits rows that exist at a time (chunk of the GEMM -> sweep -> GEMMs loop)")
    ap.add_argument("--no-compact-rows", action="store_true",
                    help="c3 only: project every row, also those without a live response token")
    ap.add_argument("--path", default="fused", choices=["fused", "split"],
                    help="fused: one sweep computes log-prob, loss and dlogits (1 read + 1 write of [T,V]); "
                         "split: forward sweep, then the backward sweep from the saved logsumexp (2 reads + 1 write)")
    ap.add_argument("--dtype", default=None, choices=["bf16", "f32"],
                    help="logits dtype instead of the workload's own (f32 at the configs[1] vocabulary: rows that two "
                         "workgroups hold in the fused sweep)")
    ap.add_argument("--upstream", type=float, default=1.0,
                    help="scalar the step multiplies the loss by before backward(), as Megatron's schedule does with "
                         "1/num_microbatches; the loss object is not told and learns it from the first backward")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--deferred-stats", action="store_true",
                    help="compute_loss(..., deferred_stats=True): the statistics are copied to the host asynchronously and "
                         "become python floats when first looked at (after the timed loop here)")
    ap.add_argument("--no-traffic", action="store_true",
                    help="do not measure the sweep's HBM traffic (two short child runs of this script under "
                         "rocprofv3 --pmc); roofline.traffic then comes from the committed profile")
    ap.add_argument("--cpu-rows", type=int, default=2048, help="rows of the CPU baseline sample")
    ap.add_argument("--seed", type=int, default=0)
    return ap.parse_args()


def make_lengths(torch, w, seed):
    gen = torch.Generator().manual_seed(seed)
    batch = w["prompts"] * w["group"]
    rlen = torch.randint(w["r_lo"], w["r_hi"] + 1, (batch, 1), generator=gen, dtype=torch.int32)
    plen = torch.ones(batch, 1, dtype=torch.int32)       # the path needs prompt_length >= 1
    p = torch.rand(w["prompts"], 1, generator=gen).repeat(1, w["group"]).reshape(batch, 1)
    rewards = torch.bernoulli(p, generator=gen)
    g = w["group"]
    if "empty_group" in w:
        rlen[w["empty_group"] * g:(w["empty_group"] + 1) * g] = 0
    if "equal_group" in w:
        rewards[w["equal_group"] * g:(w["equal_group"] + 1) * g] = 1.0
    return plen, rlen, rewards


def build_device_batch(torch, mrl, w, plen, rlen, rewards, dev, seed):
    """Synthetic batch in HBM, in the layout the training engine hands to the loss."""
    batch = plen.shape[0]
    seqlens = (plen + rlen).flatten().to(torch.int32)
    cu = torch.zeros(batch + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(seqlens, 0)
    total = int(cu[-1])
    vocab = w["vocab"]
    tdtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    padded = w.get("layout") == "padded"
    if padded:
        # [B, S, V] with S the longest sequence; rows past a sequence's end hold noise like the rest
        width = int(seqlens.max())
        total = batch * width
    logits = torch.empty(1, total, vocab, dtype=tdtype, device=dev)
    labels = torch.empty(1, total, dtype=torch.int64, device=dev)
    g = torch.Generator(device=dev).manual_seed(seed)
    chunk = 4096
    for lo in range(0, total, chunk):
        hi = min(total, lo + chunk)
        z = (torch.randn(hi - lo, vocab, generator=g, device=dev) * w["sigma"]).to(tdtype)
        logits[0, lo:hi] = z
        # a sample from softmax(z): Gumbel-max
        u = torch.rand(hi - lo, vocab, generator=g, device=dev).clamp_(1e-20, 1.0)
        labels[0, lo:hi] = torch.argmax(z.float() - torch.log(-torch.log(u)), dim=-1)
        del z, u
    resp_w = int(rlen.max())
    b = {
        "labels": labels,
        "responses": torch.zeros(batch, resp_w, dtype=torch.int32, device=dev),
        "response_length": rlen.to(dev),
        "prompt_length": plen.to(dev),
    }
    kw = dict(use_remove_padding=True, seqlens_in_batch=seqlens.to(dev), cu_seqlens_padded=cu.to(dev),
              seq_len=int(seqlens.max()))
    if padded:
        logits = logits.view(batch, width, vocab)
        b["labels"] = labels.view(batch, width)
        kw = {}
    rmask = mrl.generate_mask(b["responses"], b["response_length"])
    if w.get("loss") == "dapo":
        # configs[4]: the chunk holds the first rows of a 16-response group; rewards Bernoulli(p), p~Beta(.5,.5);
        # groups whose rewards are all equal are dropped by the dynamic-sampling filter before the loss
        full = 16
        gcpu = torch.Generator().manual_seed(seed + 7)
        while True:
            # Beta(1/2, 1/2) is the arcsine law: sin^2(pi u / 2) of a uniform u
            p = float(torch.sin(torch.rand(1, generator=gcpu) * (3.141592653589793 / 2)) ** 2)
            group_rewards = torch.bernoulli(torch.full((full, 1), p), generator=gcpu)
            if mrl.dynamic_sampling_keep_mask(group_rewards.to(dev), full).any().item():
                break
        ones = torch.ones(full, 1, device=dev)
        adv_group, _ = mrl.compute_group_norm_advantage_return(group_rewards.to(dev), ones, ones, full)
        adv = adv_group[:batch].repeat(1, resp_w) * rmask.to(torch.float32)
    else:
        adv, _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), rmask, b["response_length"], w["group"])
    b["advantages"] = adv
    # behaviour / reference log-probs: current + N(0, 0.05)
    ref_fn = mrl.LossFuncFactory.get_instance("ray_grpo", "reference")
    with torch.no_grad():
        lp0 = ref_fn.compute_loss(logits, b, forward_only=True, **kw)
    maskf = rmask.to(torch.float32)
    b["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=g, device=dev) * 0.05) * maskf
    b["ref_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=g, device=dev) * 0.05) * maskf
    return logits, b, kw, total


def cpu_baseline(torch, w, rows_target, entropy_coeff, seed, mrl=None, dev=None, path="fused"):
    """Times the oracle (torch-CPU restatement of the reference op chain) fwd+bwd on a bounded
    sample of the same workload: one group of G responses with lengths scaled so that the packed
    batch has about `rows_target` rows at the full vocabulary."""
    from oracle import advantage as o_adv
    from oracle import loss as o_loss
    from oracle import packing as o_pack
    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    gen = torch.Generator().manual_seed(seed + 1)
    group, vocab = w["group"], w["vocab"]
    mean_len = max(rows_target // group - 1, 4)
    rlen = torch.randint(max(mean_len * 3 // 4, 1), mean_len * 5 // 4 + 1, (group, 1), generator=gen, dtype=torch.int32)
    plen = torch.ones(group, 1, dtype=torch.int32)
    width, resp_w = int((plen + rlen).max()), int(rlen.max())
    ids = torch.randint(0, vocab, (group, width), generator=gen)
    mask1d = o_pack.generate_mask(ids, plen + rlen)
    labels = torch.cat([ids[:, 1:], torch.zeros(group, 1, dtype=ids.dtype)], 1)
    _, _, p_lab, seqlens, cu = o_pack.preprocess_packed_seqs(ids, labels, mask1d, 1)
    total = int(cu[-1])
    tdtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    logits = (torch.randn(1, total, vocab, generator=gen) * w["sigma"]).to(tdtype)
    rmask = o_pack.generate_mask(torch.zeros(group, resp_w), rlen)
    rewards = torch.bernoulli(torch.full((group, 1), 0.5), generator=gen)
    adv, _ = o_adv.compute_group_norm_advantage_return(rewards, rmask, rlen, group)
    b = {"labels": p_lab, "responses": torch.zeros(group, resp_w, dtype=torch.int32), "response_length": rlen,
         "prompt_length": plen, "advantages": adv}
    kw = dict(use_remove_padding=True, seqlens_in_batch=seqlens, cu_seqlens_padded=cu, seq_len=width)
    # the reference receives fp32 logits from the model's last stage
    z32 = logits.float()
    lp0 = o_loss.logprob_computer(z32, b, True, **kw)[0]
    b["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    b["ref_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen) * 0.05) * rmask
    meta = dict(clip_ratio=0.2, kl_coef=0.001, kl_penalty="low_var_kl", entropy_coeff=entropy_coeff)
    tokens = int(rlen.sum())

    def one():
        z = z32.detach().requires_grad_()
        t0 = time.perf_counter()
        loss, _ = o_loss.grpo_compute_loss(z, b, meta, **kw)
        loss.backward()
        return time.perf_counter() - t0

    for _ in range(3):
        one()
    times = sorted(one() for _ in range(5))
    med = times[len(times) // 2]
    out = {
        "value": tokens / med, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": "%d responses, %d packed rows x V=%d (fp32 up-cast), oracle fwd+bwd, median of 5 after 3 warm-ups, "
                  "%.2f s per pass" % (group, total, vocab, med),
    }
    if dev is not None:
        # the same sample through the HIP path, checked against the oracle at the full vocabulary
        z = z32.detach().requires_grad_()
        want, _ = o_loss.grpo_compute_loss(z, b, meta, **kw)
        (dz_o,) = torch.autograd.grad(want, z)
        f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.001), "kl_penalty": "low_var_kl",
                              "entropy_coeff": entropy_coeff})
        to_dev = lambda d: {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in d.items()}
        zd = logits.to(dev).requires_grad_()
        got, _ = f.compute_loss(zd, to_dev(b), fused=(path == "fused"), **to_dev(kw))
        (dz,) = torch.autograd.grad(got, zd)
        out["sample_parity"] = {
            "loss_rel_err": abs(got.item() - want.item()) / max(abs(want.item()), 1e-30),
            "dlogits_max_abs_err": (dz.float().cpu() - dz_o).abs().max().item(),
            "dlogits_max_abs": dz_o.abs().max().item(),
        }
    return out


MFMA_BF16_PEAK_TFLOPS = 2500.0


class BoardSampler:
    """Samples the shader clock and the board power from sysfs while a timed region runs (a thread that reads two
    small files every 20 ms; no GPU call).  The bf16 products run against the board's power cap, where the clock
    falls below its 2400 MHz peak: `peak_at_sclk` is the MFMA peak scaled to the clock that was actually held."""

    PEAK_SCLK_MHZ = 2400.0

    def __init__(self):
        import glob
        self.clock_files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))[:1]
        self.power_files = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"))[:1]
        self.cap_files = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"))[:1]
        self.sclk, self.power, self._stop, self._thread = [], [], False, None

    def _read_once(self):
        try:
            for f in self.clock_files:
                for line in open(f).read().splitlines():
                    if line.rstrip().endswith("*"):
                        self.sclk.append(float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip()))
            for f in self.power_files:
                self.power.append(float(open(f).read().strip()) / 1e6)
        except (OSError, ValueError, IndexError):
            pass

    def _loop(self):
        while not self._stop:
            self._read_once()
            time.sleep(0.02)

    def __enter__(self):
        import threading
        self._thread = threading.Thread(target=self._loop, daemon=True)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        self._thread.join()
        return False

    def summary(self, tflops=None):
        if not self.sclk:
            return None
        # the first samples still see the idle clock: the median of the second half is the load's
        sclk = _median(self.sclk[len(self.sclk) // 2:])
        out = {"sclk_mhz": sclk, "samples": len(self.sclk), "sclk_peak_mhz": self.PEAK_SCLK_MHZ}
        if self.power:
            out["power_w"] = _median(self.power[len(self.power) // 2:])
        try:
            out["power_cap_w"] = float(open(self.cap_files[0]).read().strip()) / 1e6
        except (OSError, ValueError, IndexError):
            pass
        if tflops is not None:
            out["peak_at_sclk"] = MFMA_BF16_PEAK_TFLOPS * sclk / self.PEAK_SCLK_MHZ
            out["frac_of_peak_at_sclk"] = tflops / out["peak_at_sclk"]
        return out


def run_lmhead(args, steps=None, warmup=None):
    """configs[3], forward part: hidden [T, 3584] ~N(0,1), W [152064, 3584] ~N(0,0.02), bf16; one step =
    log-prob + entropy + logsumexp of every token without materialising the logits."""
    import torch
    import mindspeed_rl_amd as mrl
    from mindspeed_rl_amd import lmhead
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    tokens, vocab, hdim = args.tokens, 152064, 3584
    g = torch.Generator(device=dev).manual_seed(args.seed)
    hidden = torch.randn(tokens, hdim, generator=g, device=dev).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (tokens,), generator=g, device=dev)
    for _ in range(warmup):
        mrl.lmhead_logprob(hidden, weight, labels)
    torch.cuda.synchronize()
    lmhead.kernel_events = []
    with BoardSampler() as board:
        t0 = time.perf_counter()
        for _ in range(steps):
            lp, ent, lse = mrl.lmhead_logprob(hidden, weight, labels)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    events, lmhead.kernel_events = lmhead.kernel_events, None
    ms = sum(s.elapsed_time(e) for (_, s, e, _) in events) / len(events)
    flops = 2.0 * tokens * vocab * hdim
    tflops = flops / (ms * 1e-3) / 1e12
    # spot check against a plain GEMM on a slice of the rows
    ref = torch.log_softmax(torch.nn.functional.linear(hidden[:256].float(), weight.float()), -1)
    err = (lp[:256] - ref.gather(-1, labels[:256, None]).squeeze(-1)).abs().max().item()
    result = {
        "metric": "tokens/sec for fused lm_head+logprob forward; MFMA TFLOP/s as % of bf16 dense peak",
        "value": tokens / (elapsed / steps), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": elapsed * 1e3 / steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[3] forward: hidden [%d,3584] x W [152064,3584]^T, online logsumexp, logits never "
                               "stored" % tokens, "accumulate": "f32"},
        "roofline": {"kernel": "lmhead_fwd_kernel + lmhead_finish_kernel (mrl_lmhead_logprob_fwd)", "bound": "mfma",
                     "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "flops_per_launch": flops, "avg_ms": ms},
        "max_abs_err_vs_fp32_gemm_256_rows": err,
    }
    result["roofline"]["board"] = board.summary(tflops)
    return result


def run_lmhead_train(args, steps=None, warmup=None):
    """configs[3]: GRPO loss as in configs[1] but from hidden [T, 3584] and W [152064, 3584]; backward yields
    dHidden and dW.  Logits exist for --chunk-rows rows at a time."""
    import torch
    import mindspeed_rl_amd as mrl
    from mindspeed_rl_amd import vocab_ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    w = WORKLOADS["c1"]
    vocab, hdim = w["vocab"], 3584
    plen, rlen, rewards = make_lengths(torch, w, args.seed)
    batch = plen.shape[0]
    seqlens = (plen + rlen).flatten().to(torch.int32)
    cu = torch.zeros(batch + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(seqlens, 0)
    total, tokens, resp_w = int(cu[-1]), int(rlen.sum()), int(rlen.max())
    g = torch.Generator(device=dev).manual_seed(args.seed)
    hidden = torch.randn(1, total, hdim, generator=g, device=dev).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (1, total), generator=g, device=dev)
    b = {"labels": labels, "responses": torch.zeros(batch, resp_w, dtype=torch.int32, device=dev),
         "response_length": rlen.to(dev), "prompt_length": plen.to(dev)}
    seqlens_d, cu_d = seqlens.to(dev), cu.to(dev)
    rmask = mrl.generate_mask(b["responses"], b["response_length"])
    b["advantages"], _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), rmask, b["response_length"], w["group"])
    lp_rows, _, _ = mrl.lmhead_logprob(hidden, weight, labels, want_entropy=False)
    lp0 = mrl.postprocess_packed_seqs(lp_rows, seqlens_d, cu_d, resp_w, prompt_length=b["prompt_length"])
    maskf = rmask.to(torch.float32)
    b["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=g, device=dev) * 0.05) * maskf
    ref_lp = (lp0 + torch.randn(lp0.shape, generator=g, device=dev) * 0.05) * maskf

    def step():
        h = hidden.detach().requires_grad_()
        wt = weight.detach().requires_grad_()
        loss, out = mrl.fused_lmhead_policy_loss(h, wt, b, packed=True, seqlens=seqlens_d, cu_seqlens=cu_d,
                                                 ref_log_prob=ref_lp, clip_low=0.2, clip_high=0.2,
                                                 kl_penalty="low_var_kl", kl_coef=0.001,
                                                 entropy_coeff=args.entropy_coeff, chunk_rows=args.chunk_rows,
                                                 compact_rows=not args.no_compact_rows)
        stats = out.cpu().tolist()
        dh, dw = torch.autograd.grad(loss, [h, wt])
        return loss, stats, dh, dw

    from mindspeed_rl_amd import lmhead
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    vocab_ops.kernel_events = []
    lmhead.kernel_events = []
    with BoardSampler() as board:
        t0 = time.perf_counter()
        for _ in range(steps):
            loss, stats, dh, dw = step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    events, vocab_ops.kernel_events = vocab_ops.kernel_events, None
    gemm_events, lmhead.kernel_events = lmhead.kernel_events, None
    sweep_ms = sum(s.elapsed_time(e) for (_, s, e, _) in events) / steps
    logits_ms = sum(s.elapsed_time(e) for (n, s, e, _) in gemm_events if n == "mrl_lmhead_logits") / steps
    bwd_ms = sum(s.elapsed_time(e) for (n, s, e, _) in gemm_events if n == "mrl_lmhead_logprob_bwd") / steps
    ms = elapsed * 1e3 / steps
    flops = 6.0 * total * vocab * hdim                       # forward GEMM + dHidden GEMM + dW GEMM
    tflops = flops / (ms * 1e-3) / 1e12
    del dh, dw
    # the library's kernels for the same three products of one chunk (hipBLASLt through torch), timed
    # alone and scaled to the step: a comparison figure, not part of the path
    rows = min(args.chunk_rows, total)
    h_c = hidden[0, :rows]
    z = torch.empty(rows, vocab, dtype=torch.bfloat16, device=dev)
    w_hv = weight.t().contiguous()
    dh_c = torch.empty(rows, hdim, dtype=torch.bfloat16, device=dev)
    dw32 = torch.zeros(vocab, hdim, dtype=torch.float32, device=dev)
    h_t = h_c.t().contiguous()

    def library_products():
        torch.mm(h_c, weight.t(), out=z)
        torch.mm(z, w_hv.t(), out=dh_c)
        try:
            torch.addmm(dw32, z.t(), h_t.t(), out_dtype=torch.float32, out=dw32)
        except (TypeError, RuntimeError):
            dw32.add_(torch.mm(z.t(), h_t.t()))

    library_products()
    s_ev, e_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with BoardSampler() as lib_board:
        s_ev.record()
        for _ in range(3):
            library_products()
        e_ev.record()
        torch.cuda.synchronize()
    lib_chunk_ms = s_ev.elapsed_time(e_ev) / 3
    del z, w_hv, dh_c, dw32, h_t
    result = {
        "metric": "tokens/sec for fused lm_head + logprob + GRPO loss fwd+bwd (dHidden, dW); TFLOP/s as % of bf16 dense peak",
        "value": tokens / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[3]: hidden [%d,3584] x W [152064,3584], GRPO loss as configs[1], logits only for "
                               "%d rows at a time" % (total, args.chunk_rows), "response_tokens": tokens, "accumulate": "f32",
                   "products": "hand-written gfx950 MFMA kernels (gemm_kernel: logits, dHidden, dW)",
                   "sweep": "fused_sweep_persistent_kernel in place"},
        "roofline": {"kernel": "whole step (gemm_kernel x 3 per chunk + fused_sweep_persistent_kernel)",
                     "bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "flops_per_step": flops,
                     "fused_sweeps_ms_per_step": sweep_ms, "logits_products_ms_per_step": logits_ms,
                     "backward_products_ms_per_step": bwd_ms},
        "library_products_comparison": {
            "what": "torch.mm / addmm (hipBLASLt) for the same three products of one %d-row chunk, timed alone" % rows,
            "ms_per_chunk": lib_chunk_ms, "scaled_to_step_ms": lib_chunk_ms * total / rows,
            "hand_written_products_ms_per_step": logits_ms + bwd_ms,
            "board": lib_board.summary(6.0 * rows * vocab * hdim / (lib_chunk_ms * 1e-3) / 1e12)},
        "loss": float(loss.detach()), "stats": stats[1:6],
    }
    result["roofline"]["board"] = board.summary(tflops)
    return result


# HBM bytes per launch of the dominant kernel.  Not measured by this run: the figure comes from the
# committed rocprofv3 --pmc summaries (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter
# reads for the copy probe).  Only the default workload has been profiled that way; any other
# workload, another library build (MRL_LIB_PATH) or a tuning switch (MRL_*) reports null.
PROFILED_TRAFFIC = {
    ("c1", "bf16", "fused", "mrl_fused_logprob_loss"):
        (104.05e9, "profiles/fused_sweep_persistent_kernel__c1_qwen25_grpo.md"),
    ("c1", "bf16", "split", "mrl_vocab_logprob_bwd"):
        (104.06e9, "profiles/vocab_fwd_kernel_and_bwd_chunk_kernel__c1_split_path.md"),
    ("c1", "f32", "fused", "mrl_fused_logprob_loss"):
        (208.20e9, "profiles/fused_sweep_persistent_kernel_half_rows__c1_fp32_logits.md"),
}


def _profiled_traffic(args, workload, w, path, dominant):
    """(bytes or None, where the figure comes from)."""
    if args.entropy_coeff != 0.001 or any(k.startswith("MRL_") for k in os.environ):
        return None, None
    return PROFILED_TRAFFIC.get((workload, w["dtype"], path, dominant), (None, None))


def measure_traffic(args):
    """HBM bytes per launch of the headline workload's sweep, measured now: this script is run twice more
    as a child process under `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE - one counter per run), and
    each reading of the sweep is scaled by what the same counter reads for the copy probe of known size
    in that same run.  Returns a dict, or None when rocprofv3 is missing, times out or yields nothing."""
    import csv
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(rocprof) or any(k.startswith(("ROCP_", "ROCPROF")) for k in os.environ):
        return None                                        # absent, or this process is itself being profiled
    probe_bytes = 32768 * 304128                           # what probe_copy_kernel reads, and writes
    out = {}
    work = tempfile.mkdtemp(prefix="mrl_traffic_", dir="/tmp")
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            d = os.path.join(work, counter)
            cmd = [rocprof, "--pmc", counter, "--output-format", "csv", "-d", d, "-o", "t", "--", sys.executable,
                   os.path.abspath(__file__), "--workload", "c1", "--steps", "1", "--warmup", "1", "--no-cpu-baseline",
                   "--no-traffic", "--seed", str(args.seed), "--entropy-coeff", str(args.entropy_coeff)]
            proc = subprocess.Popen(cmd, cwd="/tmp", env=dict(os.environ, TMPDIR="/tmp"), stdout=subprocess.DEVNULL,
                                    stderr=subprocess.DEVNULL, start_new_session=True)
            try:
                proc.wait(timeout=150)
            except subprocess.TimeoutExpired:
                os.killpg(proc.pid, signal.SIGKILL)
                proc.wait()
                return None
            sweep, probe = [], []
            for f in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
                for row in csv.DictReader(open(f)):
                    if row.get("Counter_Name") != counter:
                        continue
                    if "fused_sweep_persistent_kernel" in row["Kernel_Name"]:
                        sweep.append(float(row["Counter_Value"]))
                    elif "probe_copy_kernel" in row["Kernel_Name"]:
                        probe.append(float(row["Counter_Value"]))
            if not sweep or not probe:
                return None
            factor = probe_bytes / (sum(probe) / len(probe) * 1024.0)        # bytes per counted byte
            out[counter] = {"raw_KiB_per_launch": sum(sweep) / len(sweep), "copy_probe_raw_KiB": sum(probe) / len(probe),
                            "scale_factor": factor, "bytes_per_launch": sum(sweep) / len(sweep) * 1024.0 * factor,
                            "launches": len(sweep)}
    finally:
        shutil.rmtree(work, ignore_errors=True)
    return {"bytes": out["FETCH_SIZE"]["bytes_per_launch"] + out["WRITE_SIZE"]["bytes_per_launch"],
            "fetch": out["FETCH_SIZE"], "write": out["WRITE_SIZE"]}


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2] if len(xs) % 2 else 0.5 * (xs[len(xs) // 2 - 1] + xs[len(xs) // 2])


def _release(torch):
    import gc
    gc.collect()
    torch.cuda.empty_cache()


def run_sweep(args, workload, dtype=None, upstream=1.0, path=None, steps=None, warmup=None, probes=True, cpu=True,
              flush=False, deferred=None):
    """One of the logits workloads (c1, c2, c0, c4chunk) through a loss object: K timed steps bracketed by
    synchronisations, HIP events around every step (median) and around every vocabulary sweep.
    flush: a 1 GiB buffer is rewritten between the steps, outside the per-step events, so that a working
    set smaller than the last-level cache is read from HBM; the step time is then the median of the
    per-step events."""
    import torch
    import mindspeed_rl_amd as mrl
    from mindspeed_rl_amd import _lib, vocab_ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    path = args.path if path is None else path
    deferred = args.deferred_stats if deferred is None else deferred
    w = dict(WORKLOADS[workload])
    if dtype is not None and dtype != w["dtype"]:
        w["dtype"] = dtype
        w["desc"] += " [logits as %s]" % dtype
    plen, rlen, rewards = make_lengths(torch, w, args.seed)
    logits, b, kw, total = build_device_batch(torch, mrl, w, plen, rlen, rewards, dev, args.seed)
    tokens = int(rlen.sum())
    vocab = w["vocab"]
    ebytes = logits.element_size()

    if w.get("loss") == "dapo":
        f = mrl.LossFuncFactory.get_instance("ray_dapo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.2, "clip_higher_enable": True, "clip_ratio_low": 0.2,
                              "clip_ratio_high": 0.28, "token_level_loss": True, "entropy_coeff": args.entropy_coeff})
    else:
        f = mrl.LossFuncFactory.get_instance("ray_grpo", "actor")
        f.add_loss_meta_info({"clip_ratio": 0.2, "kl_ctrl": mrl.FixedKLController(0.001),
                              "kl_penalty": "low_var_kl", "entropy_coeff": args.entropy_coeff})

    # the root gradient autograd starts from, made once: torch would otherwise fill a ones tensor per step
    root = torch.full((), float(upstream), dtype=torch.float32, device=dev)

    def step():
        z = logits.detach().requires_grad_()
        loss, stats = f.compute_loss(z, b, fused=(path == "fused"), deferred_stats=deferred, **kw)
        (dz,) = torch.autograd.grad(loss, z, grad_outputs=root)
        return loss, stats, dz

    scrub = torch.empty(1 << 30, dtype=torch.uint8, device=dev) if flush else None
    rescales = f.grad_scale_state(dev).rescales
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    rescales_before = int(rescales.item())
    vocab_ops.kernel_events = []
    dz = None
    step_events = []
    stream = torch.cuda.current_stream(dev)
    with BoardSampler() as board:
        t0 = time.perf_counter()
        for _ in range(steps):
            del dz                      # the previous gradient is released before the next one is allocated
            if flush:
                scrub.fill_(1)
                torch.cuda.synchronize()
            s_ev, e_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s_ev.record(stream)
            loss, stats, dz = step()
            e_ev.record(stream)
            step_events.append((s_ev, e_ev))
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    events = vocab_ops.kernel_events
    vocab_ops.kernel_events = None
    step_ms = [s_ev.elapsed_time(e_ev) for s_ev, e_ev in step_events]
    ms_per_step = _median(step_ms) if flush else elapsed * 1e3 / steps
    hot_ms = None
    if flush:
        # the same steps back to back, caches warm, no events: what a loop over micro-batches of this size sees
        t0 = time.perf_counter()
        for _ in range(steps):
            del dz
            loss, stats, dz = step()
        torch.cuda.synchronize()
        hot_ms = (time.perf_counter() - t0) * 1e3 / steps
    graph_ms = graph_hot_ms = None
    if flush and path == "fused":
        # The same step (forward, statistics left on the device, backward) captured once into a graph and
        # replayed: one launch from the host per step instead of four plus the interpreter between them.
        # Timed like the eager steps: flushed with per-replay events (median), then back to back.
        import warnings
        warnings.filterwarnings("ignore", message=".*AccumulateGrad node's stream does not match.*")
        z_static = logits.detach().requires_grad_()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(2):
                w_loss, _w_stats = f.compute_loss(z_static, b, fused=True, deferred_stats=True, **kw)
                torch.autograd.grad(w_loss, z_static, grad_outputs=root)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g_loss, g_stats = f.compute_loss(z_static, b, fused=True, **kw)
            (g_dz,) = torch.autograd.grad(g_loss, z_static, grad_outputs=root)
        torch.cuda.synchronize()
        replay_events = []
        for _ in range(steps):
            scrub.fill_(1)
            torch.cuda.synchronize()
            s_ev, e_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s_ev.record(stream)
            graph.replay()
            e_ev.record(stream)
            replay_events.append((s_ev, e_ev))
        torch.cuda.synchronize()
        graph_ms = _median([a.elapsed_time(c) for a, c in replay_events])
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_hot_ms = (time.perf_counter() - t0) * 1e3 / steps
        # the replayed step is the eager step: same loss, same gradient, same statistics
        if not (float(g_loss.detach()) == float(loss.detach()) and torch.equal(g_dz, dz)
                and all(g_stats[k] == float(v) for k, v in stats.items())):
            raise RuntimeError("graph replay differs from the eager step")
        del graph, g_dz

    def avg_ms(name):
        ts = [s.elapsed_time(e) for (n, s, e, _) in events if n == name]
        return sum(ts) / len(ts) if ts else None

    live_rows = tokens                                    # rows with a non-zero mask / incoming gradient
    dead_rows = total - live_rows
    row_bytes = vocab * ebytes
    # algorithmic HBM bytes per launch: reads of the rows that are needed (the split path's forward is
    # handed the rows inside the response windows, like the fused sweep) + writes of every dlogits row
    kernel_bytes = {
        "mrl_vocab_logprob_fwd": live_rows * row_bytes,
        "mrl_vocab_logprob_bwd": live_rows * 2 * row_bytes + dead_rows * row_bytes,
        "mrl_fused_logprob_loss": live_rows * 2 * row_bytes + dead_rows * row_bytes,
    }
    # the kernel each entry point dispatches to for this shape (csrc/row_sweep.hip, csrc/vocab_logprob.hip)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    wide = row_bytes > 19 * 1024 * 16                      # a row that two workgroups hold
    persistent = wide or total > 2 * cus
    chunked = row_bytes >= 16384 and row_bytes % 16 == 0
    kernel_symbol = {"mrl_vocab_logprob_fwd": "vocab_fwd_kernel",
                     "mrl_vocab_logprob_bwd": "bwd_chunk_kernel" if chunked else "vocab_bwd_kernel",
                     "mrl_fused_logprob_loss": ("fused_sweep_persistent_kernel" + (" (half rows)" if wide else ""))
                     if persistent else "fused_sweep_kernel"}
    kernels = {}
    for name, nbytes in kernel_bytes.items():
        ms = avg_ms(name)
        if ms is not None:
            gbps = nbytes / (ms * 1e-3) / 1e9
            kernels[name] = {"symbol": kernel_symbol[name], "avg_ms": ms, "GBps": gbps, "frac": gbps / HBM_PEAK_GBPS,
                             "bytes_per_launch": nbytes}
    dominant = max(kernels, key=lambda n: kernels[n]["avg_ms"])
    step_bytes = sum(k["bytes_per_launch"] for k in kernels.values())
    step_gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    # the split path's 3 passes (read, read, write) are the reference accounting of the task; the fused
    # path needs only 2 of them, so the same step is also quoted against that 3-pass byte count
    three_pass_bytes = total * row_bytes + live_rows * 2 * row_bytes + dead_rows * row_bytes
    three_pass_gbps = three_pass_bytes / (ms_per_step * 1e-3) / 1e9
    traffic, traffic_source = _profiled_traffic(args, workload, w, path, dominant)

    result = {
        "metric": "tokens/sec for logprob+GRPO loss fwd+bwd; achieved HBM GB/s as % of peak",
        "value": tokens / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w["dtype"],
        "data": "synthetic",
        "config": {
            "workload": w["desc"], "responses": int(plen.shape[0]), "layout": w.get("layout", "packed"),
            "packed_rows": total, "response_tokens": tokens,
            "vocab": vocab, "accumulate": "f32", "loss_kind": w.get("loss", "grpo: clip 0.2, low_var_kl 0.001"),
            "entropy_coeff": args.entropy_coeff, "loss": "token-mean", "path": path,
            # the scalar autograd starts the backward from; the loss object is not told
            "upstream": upstream,
            "caches_flushed_between_steps": bool(flush),
            "deferred_stats": bool(deferred),
        },
        "roofline": {
            "kernel": "%s (%s)" % (kernels[dominant]["symbol"], dominant), "bound": "hbm",
            "achieved": kernels[dominant]["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": kernels[dominant]["frac"], "traffic": traffic,
            "traffic_source": {"measured_this_run": False, "from_committed_profile": traffic_source},
            "bytes_per_launch": kernels[dominant]["bytes_per_launch"], "avg_ms": kernels[dominant]["avg_ms"],
        },
        "ms_per_step_median": _median(step_ms),
        "ms_per_step_mean_wall": elapsed * 1e3 / steps,
        "ms_per_step_hot": hot_ms,
        "ms_per_step_graph_replay": graph_ms,
        "ms_per_step_hot_graph_replay": graph_hot_ms,
        "kernels": kernels,
        "step_hbm": {"GBps": step_gbps, "frac": step_gbps / HBM_PEAK_GBPS, "algorithmic_bytes_per_step": step_bytes},
        # NOT a roofline fraction: the step's time applied to the bytes a 3-pass (read, read, write)
        # implementation would move, so that the fused and the split path can be compared on one denominator
        "comparison_on_three_pass_bytes": {"bytes": three_pass_bytes, "equivalent_GBps": three_pass_gbps},
        "rescale_passes_in_timed_steps": int(rescales.item()) - rescales_before if path == "fused" else None,
        "stats": {k: float(v) for k, v in stats.items()},
        "loss": float(loss.detach()),
        "board": board.summary(),
    }
    host_copy = None
    if cpu == "whole":
        to_host = lambda d: {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in d.items()}
        host_copy = (logits.detach().cpu(), to_host(b), to_host(kw), tokens)
    del dz, scrub, logits, b
    _release(torch)
    if probes:
        result["measured_ceiling"] = bandwidth_ceilings(torch, _lib, dev)
        # a read+write stream of R read bytes and W written bytes cannot beat R/read + W/write on this box
        best_copy = max(result["measured_ceiling"]["copy_GBps"], result["measured_ceiling"]["stream_copy_GBps"])
        for k in kernels.values():
            k["frac_of_measured_copy"] = k["GBps"] / best_copy
        result["roofline"]["frac_of_measured_copy_ceiling"] = kernels[dominant]["GBps"] / best_copy
    if cpu == "whole":
        result["cpu_baseline"] = cpu_baseline_whole(torch, w, host_copy, args.entropy_coeff, float(result["loss"]))
    elif cpu:
        result["cpu_baseline"] = cpu_baseline(torch, w, args.cpu_rows, args.entropy_coeff, args.seed, mrl, dev, path)
    return result


def cpu_baseline_whole(torch, w, host_copy, entropy_coeff, gpu_loss):
    """The oracle on the WHOLE batch of a workload that fits the host (configs[0]): the very logits and
    batch the GPU steps ran on, forward + backward, median of 5 after 2 warm-ups."""
    from oracle import loss as o_loss
    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    logits, b, kw, tokens = host_copy
    meta = dict(clip_ratio=0.2, kl_coef=0.001, kl_penalty="low_var_kl", entropy_coeff=entropy_coeff)
    z32 = logits.float()

    def one():
        z = z32.detach().requires_grad_()
        t0 = time.perf_counter()
        loss, _ = o_loss.grpo_compute_loss(z, b, meta, **kw)
        loss.backward()
        return time.perf_counter() - t0, float(loss.detach())

    for _ in range(2):
        one()
    runs = sorted(one() for _ in range(5))
    med, cpu_loss = runs[len(runs) // 2]
    return {"value": tokens / med, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": "the whole batch: %d responses, %d packed rows x V=%d, oracle fwd+bwd, median of 5 after 2 warm-ups, "
                      "%.3f s per pass" % (b["responses"].shape[0], logits.shape[1], logits.shape[-1], med),
            "loss_rel_err_gpu_vs_oracle": abs(gpu_loss - cpu_loss) / max(abs(cpu_loss), 1e-30)}


def bandwidth_ceilings(torch, _lib, dev):
    """Practical ceilings on this box: with the sweeps' access pattern (one workgroup per 152064-entry bf16
    row) and with the pattern the HBM system serves best (one vector per thread, small workgroups)."""
    probe_rows, probe_row_bytes = 32768, 304128
    nbytes = probe_rows * probe_row_bytes
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    dst = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    ceilings = {}
    for mode, name, passes in ((0, "read_GBps", 1), (1, "write_GBps", 1), (2, "copy_GBps", 2),
                               (3, "stream_read_GBps", 1), (4, "stream_write_GBps", 1), (5, "stream_copy_GBps", 2)):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(2):
            _lib.call("mrl_bandwidth_probe", mode, src.data_ptr(), dst.data_ptr(), probe_rows, probe_row_bytes,
                      _lib.stream(dev))
        s.record()
        for _ in range(5):
            _lib.call("mrl_bandwidth_probe", mode, src.data_ptr(), dst.data_ptr(), probe_rows, probe_row_bytes,
                      _lib.stream(dev))
        e.record()
        torch.cuda.synchronize()
        ceilings[name] = passes * nbytes * 5 / (s.elapsed_time(e) * 1e-3) / 1e9
    # the runtime's own device-to-device copy of the same bytes (Tensor.copy_ -> hipMemcpyAsync)
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(2):
        dst.copy_(src)
    s.record()
    for _ in range(5):
        dst.copy_(src)
    e.record()
    torch.cuda.synchronize()
    ceilings["runtime_d2d_copy_GBps"] = 2 * nbytes * 5 / (s.elapsed_time(e) * 1e-3) / 1e9
    return ceilings


# ----------------------------------------------------------------------------------------- configs[4], whole
C4 = dict(prompts=8, group=16, r_lo=8192, r_hi=32768, vocab=129280, sigma=3.0)


def make_c4_batch(torch, mrl, dev, seed):
    """The experience batch of configs[4] without its logits: 8 prompts x 16 responses, R ~ U[8192, 32768],
    1-token prompts, rewards Bernoulli(p), p ~ Beta(1/2, 1/2) per prompt; the dynamic-sampling filter
    (workers/dynamic_sampling.py:81-86 of the reference) drops the groups whose rewards are all equal
    BEFORE anything else sees the batch; advantages are the group-normalised rewards of the kept groups.
    The seed is advanced until at least one group is dropped and at least three are kept.
    Returns (batch on the device, kept row indices, rows before the filter)."""
    n_all = C4["prompts"] * C4["group"]
    while True:
        gen = torch.Generator().manual_seed(seed)
        rlen = torch.randint(C4["r_lo"], C4["r_hi"] + 1, (n_all, 1), generator=gen, dtype=torch.int32)
        # Beta(1/2, 1/2) is the arcsine law: sin^2(pi u / 2) of a uniform u
        p = torch.sin(torch.rand(C4["prompts"], 1, generator=gen) * (3.141592653589793 / 2)) ** 2
        rewards = torch.bernoulli(p.repeat(1, C4["group"]).reshape(n_all, 1), generator=gen)
        keep = mrl.dynamic_sampling_keep(rewards.flatten().to(dev), C4["group"])
        if 3 * C4["group"] <= len(keep) < n_all:
            break
        seed += 1000
    rlen, rewards = rlen[keep], rewards[keep]
    n_seq, resp_w = len(keep), int(rlen.max())
    full = {
        "responses": torch.zeros(n_seq, resp_w, dtype=torch.int32, device=dev),
        "response_length": rlen.to(dev),
        "prompt_length": torch.ones(n_seq, 1, dtype=torch.int32, device=dev),
    }
    rmask = mrl.generate_mask(full["responses"], full["response_length"])
    full["advantages"], _ = mrl.compute_group_norm_advantage_return(rewards.to(dev), rmask, full["response_length"],
                                                                    C4["group"])
    return full, keep, n_all


def c4_micro_batch_inputs(torch, mrl, mb, dev, gen, ref_fn):
    """Logits, labels and old log-probs of one micro-batch, made on the device: packed [1, T, V] bf16
    logits ~N(0, 3), uniform labels, old = current log-prob + N(0, 0.05).  Returns (logits, kwargs)."""
    vocab = C4["vocab"]
    seqlens = (mb["prompt_length"] + mb["response_length"]).flatten().to(torch.int32)
    cu = torch.zeros(seqlens.numel() + 1, dtype=torch.int32, device=dev)
    cu[1:] = torch.cumsum(seqlens, 0)
    total = int(cu[-1].item())
    logits = torch.empty(1, total, vocab, dtype=torch.bfloat16, device=dev)
    for lo in range(0, total, 8192):
        hi = min(total, lo + 8192)
        logits[0, lo:hi] = torch.randn(hi - lo, vocab, generator=gen, device=dev, dtype=torch.bfloat16) * C4["sigma"]
    mb["labels"] = torch.randint(0, vocab, (1, total), generator=gen, device=dev)
    kw = dict(use_remove_padding=True, seqlens_in_batch=seqlens, cu_seqlens_padded=cu, seq_len=int(seqlens.max().item()))
    with torch.no_grad():
        lp0 = ref_fn.compute_loss(logits, mb, forward_only=True, **kw)
    maskf = mrl.generate_mask(mb["responses"], mb["response_length"]).to(torch.float32)
    mb["old_log_prob"] = (lp0 + torch.randn(lp0.shape, generator=gen, device=dev) * 0.05) * maskf
    return logits, kw, total


def run_c4(args, steps=None, warmup=None):
    """configs[4] as the reference runs it (models/base/base_training_engine.py:160-208 with use_dynamic_bsz):
    the filtered batch is cut into token-budget micro-batches by the Karmarkar-Karp partitioner, and every
    micro-batch goes through ONE DAPO loss object with use_dynamic_bsz / actual_micro_batch_size and
    (loss / n_micro).backward().  One step = all micro-batches of the batch; the logits of a micro-batch
    (up to 17 GB) are generated on the device right before it and are not part of the timed regions."""
    import torch
    import mindspeed_rl_amd as mrl
    from mindspeed_rl_amd import vocab_ops
    from mindspeed_rl_amd import seqlen_balancing as bal
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    full, keep, n_all = make_c4_batch(torch, mrl, dev, args.seed)
    n_seq = len(keep)
    batches, parts = bal.split_batches_with_dynamic_bsz(full, args.token_budget, None)
    n_micro = len(batches)
    f = mrl.LossFuncFactory.get_instance("ray_dapo", "actor")
    f.add_loss_meta_info({"clip_ratio": 0.2, "clip_higher_enable": True, "clip_ratio_low": 0.2,
                          "clip_ratio_high": 0.28, "token_level_loss": True, "entropy_coeff": args.entropy_coeff})
    ref_fn = mrl.LossFuncFactory.get_instance("ray_grpo", "reference")
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    rescales = f.grad_scale_state(dev).rescales
    vocab, row_bytes = C4["vocab"], C4["vocab"] * 2
    tokens = int(full["response_length"].sum().item())

    def one_pass(record):
        """All micro-batches once; returns (seconds inside the timed regions, per-micro-batch records)."""
        spent, rows_seen, micro = 0.0, 0, []
        for mb in batches:
            mb = dict(mb)
            logits, kw, total = c4_micro_batch_inputs(torch, mrl, mb, dev, gen, ref_fn)
            z = logits.requires_grad_()
            torch.cuda.synchronize()
            if record:
                vocab_ops.kernel_events = []
            t0 = time.perf_counter()
            loss, stats = f.compute_loss(z, mb, use_dynamic_bsz=True, actual_micro_batch_size=n_seq / n_micro,
                                         index=None, **kw)
            (loss / n_micro).backward()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            spent += dt
            rows_seen += total
            if record:
                events, vocab_ops.kernel_events = vocab_ops.kernel_events, None
                sweep_ms = sum(s.elapsed_time(e) for (n, s, e, _) in events if n == "mrl_fused_logprob_loss")
                live = int(mb["response_length"].sum().item())
                nbytes = live * 2 * row_bytes + (total - live) * row_bytes
                micro.append({"sequences": int(mb["response_length"].numel()), "rows": total, "step_ms": dt * 1e3,
                              "sweep_ms": sweep_ms, "sweep_GBps": nbytes / (sweep_ms * 1e-3) / 1e9,
                              "sweep_bytes": nbytes, "loss": float(loss.detach())})
            del z, logits, loss
        return spent, rows_seen, micro

    for _ in range(warmup):
        one_pass(False)
    torch.cuda.synchronize()
    rescales_before = int(rescales.item())
    spent, micro = 0.0, []
    for _ in range(steps):
        dt, rows_seen, m = one_pass(True)
        spent += dt
        micro += m
    ms_per_step = spent * 1e3 / steps
    sweep_ms = sum(m["sweep_ms"] for m in micro)
    sweep_bytes = sum(m["sweep_bytes"] for m in micro)
    gbps = sweep_bytes / (sweep_ms * 1e-3) / 1e9
    per_micro = sorted(m["sweep_GBps"] for m in micro)
    result = {
        "metric": "tokens/sec for logprob+DAPO loss fwd+bwd; achieved HBM GB/s as % of peak",
        "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "configs[4]: 8x16 responses, R~U[8192,32768], V=129280 bf16, DAPO clip-higher 0.2/0.28, no KL, "
                        "token-level loss; dynamic-sampling filter, then Karmarkar-Karp micro-batches of at most %d "
                        "tokens through one loss object, (loss / n_micro).backward()" % args.token_budget,
            "responses_before_filter": n_all, "responses_kept": n_seq, "groups_dropped": (n_all - n_seq) // C4["group"],
            "micro_batches": n_micro, "token_budget": args.token_budget, "packed_rows": rows_seen,
            "response_tokens": tokens, "vocab": vocab, "accumulate": "f32", "entropy_coeff": args.entropy_coeff,
            "timed": "compute_loss + backward of every micro-batch (its logits are generated before, untimed)",
        },
        "roofline": {
            "kernel": "fused_sweep_persistent_kernel (mrl_fused_logprob_loss), all micro-batches", "bound": "hbm",
            "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": None,
            "bytes_per_launch": sweep_bytes / len(micro), "avg_ms": sweep_ms / len(micro),
            "per_micro_batch_GBps": {"min": per_micro[0], "median": _median(per_micro), "max": per_micro[-1]},
        },
        "rescale_passes_in_timed_steps": int(rescales.item()) - rescales_before,
        "rescale_passes_in_all": int(rescales.item()),
        "micro_batch_rows": {"min": min(m["rows"] for m in micro), "max": max(m["rows"] for m in micro)},
        "micro_batch_step_ms": {"min": min(m["step_ms"] for m in micro), "median": _median([m["step_ms"] for m in micro]),
                                "max": max(m["step_ms"] for m in micro)},
        "loss": sum(m["loss"] for m in micro[-n_micro:]) / n_micro,
    }
    del batches, full
    _release(torch)
    return result


def _compact(r):
    """What other_workloads keeps of a result line."""
    roof = r["roofline"]
    out = {"ms_per_step": r["ms_per_step"], "value": r["value"], "unit": r["unit"], "steps": r["steps"],
           "workload": r["config"]["workload"],
           "roofline": {"kernel": roof["kernel"], "bound": roof["bound"], "achieved": roof["achieved"],
                        "unit": roof["unit"], "frac": roof["frac"], "avg_ms": roof.get("avg_ms")}}
    for key in ("ms_per_step_median", "ms_per_step_hot", "ms_per_step_graph_replay", "ms_per_step_hot_graph_replay",
                "cpu_baseline", "rescale_passes_in_timed_steps", "library_products_comparison",
                "micro_batch_rows", "micro_batch_step_ms"):
        if r.get(key) is not None:
            out[key] = r[key]
    for key in ("per_micro_batch_GBps", "fused_sweeps_ms_per_step", "logits_products_ms_per_step",
                "backward_products_ms_per_step", "board"):
        if key in roof:
            out["roofline"][key] = roof[key]
    for key in ("micro_batches", "responses_kept", "groups_dropped", "caches_flushed_between_steps"):
        if key in r["config"]:
            out[key] = r["config"][key]
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives exist on this path); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    import mindspeed_rl_amd as mrl  # noqa: F401  (fails loudly if the library is not built)
    from mindspeed_rl_amd import _lib
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    _lib.load()
    cpu = not args.no_cpu_baseline
    if args.workload == "c3fwd":
        result = run_lmhead(args)
    elif args.workload == "c3":
        result = run_lmhead_train(args)
    elif args.workload == "c4":
        result = run_c4(args)
    elif args.workload == "c0":
        result = run_sweep(args, "c0", dtype=args.dtype, upstream=args.upstream, cpu="whole" if cpu else False, flush=True)
    elif args.workload != "all":
        result = run_sweep(args, args.workload, dtype=args.dtype, upstream=args.upstream, cpu=cpu)
    else:
        # the headline first and alone on the card, then a few steps of everything else
        result = run_sweep(args, "c1", dtype=args.dtype, upstream=args.upstream, cpu=cpu)
        k, others = args.other_steps, {}
        others["c0"] = _compact(run_sweep(args, "c0", steps=max(k, 20), warmup=3, probes=False,
                                          cpu="whole" if cpu else False, flush=True, deferred=False))
        # the same with the statistics fetched lazily (no synchronisation between forward and backward)
        lazy = run_sweep(args, "c0", steps=max(k, 20), warmup=3, probes=False, cpu=False, flush=True, deferred=True)
        others["c0"]["ms_per_step_deferred_stats"] = lazy["ms_per_step"]
        others["c0"]["ms_per_step_hot_deferred_stats"] = lazy["ms_per_step_hot"]
        others["c2"] = _compact(run_sweep(args, "c2", steps=k, warmup=1, probes=False, cpu=False))
        others["c4"] = _compact(run_c4(args, steps=1, warmup=1))
        others["f32"] = _compact(run_sweep(args, "c1", dtype="f32", steps=k, warmup=1, probes=False, cpu=False))
        others["upstream0.25"] = _compact(run_sweep(args, "c1", upstream=0.25, steps=k, warmup=2, probes=False, cpu=False))
        others["c3fwd"] = _compact(run_lmhead(args, steps=k, warmup=1))
        others["c3"] = _compact(run_lmhead_train(args, steps=max(1, k - 1), warmup=1))
        result["other_workloads"] = others
        # the sweep's HBM traffic, measured now (the card is free again: children of this process run it)
        if not args.no_traffic and args.dtype in (None, "bf16") and args.path == "fused":
            measured = measure_traffic(args)
            if measured is not None:
                result["roofline"]["traffic"] = measured["bytes"]
                result["roofline"]["traffic_source"] = {
                    "measured_this_run": True,
                    "method": "two child runs of `bench.py --workload c1 --steps 1 --warmup 1` under rocprofv3 --pmc "
                              "(FETCH_SIZE, then WRITE_SIZE), each scaled by the copy probe of the same run",
                    "fetch": measured["fetch"], "write": measured["write"]}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
