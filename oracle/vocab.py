"""Oracle (test infrastructure): per-token log-probability and entropy over the vocabulary.

Restates, op for op and at tensor-parallel size 1 (every TP all-reduce is the identity):

* Megatron-LM ``core_v0.12.1`` ``megatron/core/tensor_parallel/cross_entropy.py``
  (``VocabParallelCrossEntropy`` + ``_VocabParallelCrossEntropy``) - not vendored in the
  reference; call sites ``cli/train_grpo.py:327,349`` and
  ``mindspeed_rl/utils/compute.py:50``.  PARITY UNPINNED against the real Megatron code
  (the reference's tests mock it); pinned against textbook closed forms in ``tests/``.
* ``mindspeed_rl/utils/compute.py:29-51``  (``compute_log_probs``)
* ``mindspeed_rl/utils/compute.py:54-97``  (``_VocabParallelEntropy``)

The cost structure of the reference is kept on purpose (clone, fp32 up-cast, one torch op
per step, softmax saved for backward) because the benchmark times this code as the CPU
baseline.
"""
import torch


class _MegatronCrossEntropyTP1(torch.autograd.Function):
    """Megatron ``_VocabParallelCrossEntropy`` with a one-rank tensor-parallel group."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, label_smoothing=0.0):
        if label_smoothing != 0.0:
            raise NotImplementedError("the reference never passes label smoothing")
        # calculate_logits_max: up-cast, row max
        z = vocab_parallel_logits.float()
        row_max = torch.max(z, dim=-1)[0]
        # calculate_predicted_logits: in-place shift, masked gather, in-place exp, row sum
        z -= row_max.unsqueeze(dim=-1)
        vocab = z.size(-1)
        out_of_range = (target < 0) | (target >= vocab)
        safe_target = target.clone()
        safe_target[out_of_range] = 0
        z2d = z.view(-1, vocab)
        flat_target = safe_target.view(-1)
        rows = torch.arange(start=0, end=z2d.size(0), device=z2d.device)
        picked = z2d[rows, flat_target].clone().contiguous().view_as(target)
        picked[out_of_range] = 0.0
        torch.exp(z, out=z)
        sum_exp = z.sum(dim=-1)
        # calculate_cross_entropy_loss
        loss = torch.log(sum_exp) - picked
        z.div_(sum_exp.unsqueeze(dim=-1))          # z now holds the softmax
        ctx.save_for_backward(z, out_of_range, flat_target)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        softmax, out_of_range, flat_target = ctx.saved_tensors
        vocab = softmax.size(-1)
        grad = softmax                              # Megatron re-uses the saved buffer
        g2d = grad.view(-1, vocab)
        rows = torch.arange(start=0, end=g2d.size(0), device=g2d.device)
        g2d[rows, flat_target] -= 1.0 - out_of_range.view(-1).float()
        grad.mul_(grad_output.unsqueeze(dim=-1))
        return grad, None, None


def megatron_vocab_parallel_cross_entropy(vocab_parallel_logits, target, label_smoothing=0.0):
    """Per-token cross entropy; like Megatron's, it may clobber a fp32 ``vocab_parallel_logits``."""
    return _MegatronCrossEntropyTP1.apply(vocab_parallel_logits, target, label_smoothing)


def compute_log_probs(logits, labels, **kwargs):
    """``mindspeed_rl/utils/compute.py:29-51``: clone both, negate Megatron's CE."""
    logits = logits.clone()
    labels = labels.clone()
    return -megatron_vocab_parallel_cross_entropy(vocab_parallel_logits=logits, target=labels)


class _EntropyTP1(torch.autograd.Function):
    """``mindspeed_rl/utils/compute.py:54-85`` with the three TP all-reduces removed.

    Runs in the dtype of its input (the reference does not up-cast here)."""

    @staticmethod
    def forward(ctx, z):
        z_max = z.max(dim=-1, keepdim=True).values
        shifted = z - z_max
        e = shifted.exp_()
        sum_e = e.sum(dim=-1, keepdim=True)
        p = e.div_(sum_e)
        p_dot_z = (p * z).sum(dim=-1, keepdim=True)
        entropy = z_max + sum_e.log() - p_dot_z
        ctx.save_for_backward(z, p, p_dot_z)
        return entropy.squeeze(dim=-1)

    @staticmethod
    def backward(ctx, grad_output):
        z, p, p_dot_z = ctx.saved_tensors
        # the reference mutates its saved tensors and then restores the logits; the
        # oracle keeps the same arithmetic order without the aliasing
        centred = z - p_dot_z
        grad = p * centred
        grad = grad * grad_output.unsqueeze(dim=-1)
        return -grad


def vocab_parallel_entropy(vocab_parallel_logits):
    """``mindspeed_rl/utils/compute.py:88-97``."""
    return _EntropyTP1.apply(vocab_parallel_logits)


def logprob_entropy_fp64(logits, labels):
    """Independent fp64 brute-force closed form used to pin the two functions above."""
    z = logits.double()
    lse = torch.logsumexp(z, dim=-1)
    logp = z.gather(-1, labels.long().unsqueeze(-1)).squeeze(-1) - lse
    p = torch.softmax(z, dim=-1)
    ent = lse - (p * z).sum(-1)
    return logp, ent, lse


def lmhead_logprob_entropy(hidden, weight, labels, inv_temperature=1.0):
    """Oracle of the fused lm_head path: the logits are the fp32 product of the bf16 operands
    (``F.linear`` on the up-cast tensors, no rounding of the logits to bf16), followed by the two
    functions above.  The reference materialises bf16 logits in ``GPTModel.output_layer`` (external
    Megatron code) before ``compute_log_probs`` up-casts them; a kernel that never stores the logits
    has no reason to round them, so the comparison is made on the fp32 product."""
    logits = torch.nn.functional.linear(hidden.float(), weight.float()) * inv_temperature
    return compute_log_probs(logits, labels), vocab_parallel_entropy(logits), torch.logsumexp(logits, -1)
