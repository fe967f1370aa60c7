"""The entry point that allocates nothing: mrl_lmhead_logprob_fwd_static keeps its partial
statistics in a static device array of the library instead of a caller's workspace."""
import pytest
import torch

from mindspeed_rl_amd import _lib

pytestmark = pytest.mark.gpu


def _case(dev, seed, tokens, vocab, hdim):
    g = torch.Generator(device=dev).manual_seed(seed)
    hidden = torch.randn(tokens, hdim, generator=g, device=dev).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=dev) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (tokens,), generator=g, device=dev)
    return hidden, weight, labels


def _outputs(dev, tokens):
    return [torch.full((tokens,), float("nan"), dtype=torch.float32, device=dev) for _ in range(3)]


def test_static_scratch_entry_point_matches_the_workspace_one():
    """Through the C ABI, two calls in a row, the second with a smaller input: log-prob, entropy and
    logsumexp are bit-identical to mrl_lmhead_logprob_fwd's (same kernels, same merge order), and a
    token count beyond the static array is rejected before anything is launched."""
    assert torch.cuda.is_available()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.load()
    limit = lib.mrl_lmhead_static_max_tokens()
    assert limit == 65536
    stream = _lib.stream(dev)
    for seed, tokens, vocab, hdim in ((1, 1500, 4096 + 24, 256), (2, 300, 1000, 128)):
        hidden, weight, labels = _case(dev, seed, tokens, vocab, hdim)
        want = _outputs(dev, tokens)
        ws_bytes = lib.mrl_lmhead_workspace_bytes(tokens, vocab)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        _lib.call("mrl_lmhead_logprob_fwd", hidden.data_ptr(), weight.data_ptr(), tokens, vocab, hdim, labels.data_ptr(),
                  _lib.I64, 1.25, want[0].data_ptr(), want[1].data_ptr(), want[2].data_ptr(), workspace.data_ptr(),
                  ws_bytes, stream)
        got = _outputs(dev, tokens)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(dev)
        _lib.call("mrl_lmhead_logprob_fwd_static", hidden.data_ptr(), weight.data_ptr(), tokens, vocab, hdim,
                  labels.data_ptr(), _lib.I64, 1.25, got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(), stream)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        for a, b in zip(got, want):
            assert torch.isfinite(b).all().item() and torch.equal(a, b)
        # against a plain fp32 GEMM + log-softmax of the same operands
        ref = torch.log_softmax(torch.nn.functional.linear(hidden.float(), weight.float()) * 1.25, -1)
        assert (got[0] - ref.gather(-1, labels[:, None])[:, 0]).abs().max().item() < 1e-3
        assert (got[1] + (ref.exp() * ref).sum(-1)).abs().max().item() < 1e-3
    # beyond the static array: refused with a message, nothing launched, outputs untouched
    hidden, weight, labels = _case(dev, 3, 8, 256, 64)
    out = _outputs(dev, 8)
    rc = lib.mrl_lmhead_logprob_fwd_static(hidden.data_ptr(), weight.data_ptr(), limit + 1, 256, 64, labels.data_ptr(),
                                           _lib.I64, 1.0, out[0].data_ptr(), None, None, stream)
    assert rc == -2 and b"65536" in lib.mrl_last_error()
    torch.cuda.synchronize()
    assert torch.isnan(out[0]).all().item()
    assert lib.mrl_lmhead_logprob_fwd_static(None, None, 0, 256, 64, None, _lib.I64, 1.0, None, None, None, None) == 0
