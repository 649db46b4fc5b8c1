"""Arg-max token + confidence kernel against the oracle's restatement of the reference transfer rule
(nano-vdllm/model_runner.py:2279-2296).  Tokens are index-exact (first maximum); confidences are fp32 results
of a differently ordered sum, compared at 2e-5 relative (and against a float64 evaluation)."""
import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu
REL = 2e-5


def _check(logits, device, picks=None):
    want_tok, want_conf = O.argmax_confidence(logits, picks)
    tok, conf = ops.argmax_confidence(logits.to(device), None if picks is None else picks.to(device))
    assert torch.equal(tok.cpu(), want_tok)
    rows = logits.reshape(-1, logits.shape[-1]).double()
    exact = torch.exp(rows.gather(-1, want_tok.reshape(-1, 1)).squeeze(-1) - torch.logsumexp(rows, -1)).view_as(want_conf)
    got = conf.cpu().double()
    assert torch.allclose(got, want_conf.double(), rtol=REL, atol=1e-30)
    assert torch.allclose(got, exact, rtol=REL, atol=1e-30)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("R,V", [(7, 64), (33, 1000), (16, 126464)])
def test_argmax_confidence_matches_oracle(device, dtype, R, V):
    g = torch.Generator().manual_seed(R * 1000 + V)
    _check((torch.randn(R, V, generator=g) * 3).to(dtype), device)


def test_peaked_rows_ties_and_minus_inf(device):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 512, generator=g).to(torch.bfloat16)
    x[0, 100] = 30.0                                  # confidence ~ 1
    x[1, [7, 300, 301]] = 9.0                         # three equal maxima: the first index wins
    x[2, :] = 0.5                                     # uniform row: token 0, confidence 1 / V
    x[3, 200:] = float("-inf")                        # masked-out vocabulary tail
    x[4, :] = float("-inf"); x[4, 411] = -3.0         # a single finite entry: confidence 1
    x[5, 0] = 5.0; x[5, 511] = 5.0                    # tie between the first and the last column
    _check(x, device)
    tok, conf = ops.argmax_confidence(x.to(device))
    assert tok.tolist() == [100, 7, 0, int(x[3].float().argmax()), 411, 0]
    assert abs(conf[2].item() - 1 / 512) < 1e-8 and abs(conf[4].item() - 1.0) < 1e-6


def test_batched_shape_tail_columns_and_picks(device):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 5, 1000, generator=g)                       # [B, L, V] logits as the engine passes them
    tok, conf = ops.argmax_confidence(x.to(device))
    want_tok, want_conf = O.argmax_confidence(x)
    assert tok.shape == (3, 5) and torch.equal(tok.cpu(), want_tok)
    assert torch.allclose(conf.cpu(), want_conf, rtol=REL, atol=0)
    picks = torch.randint(0, 1000, (3, 5), generator=g)            # Gumbel picks drawn by the caller
    _check(x, device, picks)

    # V = 1001 fp32 columns inside rows of stride 1004 (16-byte aligned): the last column is a ragged tail
    import ctypes
    from acache_amd import _lib
    xs = torch.randn(15, 1004, generator=g)
    xs[0, 1000] = 50.0                                             # maximum inside the tail
    dev = xs.to(device)
    out_t = torch.empty(15, dtype=torch.int64, device=device)
    out_c = torch.empty(15, dtype=torch.float32, device=device)
    rc = _lib.load().acache_argmax_confidence(out_t.data_ptr(), out_c.data_ptr(), dev.data_ptr(), None, 15, 1001, 1004, 2,
                                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    want_tok, want_conf = O.argmax_confidence(xs[:, :1001])
    assert torch.equal(out_t.cpu(), want_tok) and out_t[0].item() == 1000
    assert torch.allclose(out_c.cpu(), want_conf, rtol=REL, atol=0)


def test_argument_errors(device):
    x = torch.randn(4, 50, device=device).to(torch.bfloat16)      # 100-byte rows: not 16-byte aligned
    with pytest.raises(ValueError, match="aligned"):
        ops.argmax_confidence(x)


def _commit_rule(blocks, proposal, conf, mask_id, threshold):
    """The commit rule in tensor operations (the formulation of ModelRunner.get_transfer_index and of the write that
    follows it): returns the new blocks and the number of rows that committed."""
    committable = (blocks == mask_id) & (proposal != mask_id)
    c = torch.where(committable, conf, torch.full_like(conf, -float("inf")))
    accept = (c >= threshold) & committable
    stuck = committable.any(dim=1) & ~accept.any(dim=1)
    forced = torch.zeros_like(accept).scatter_(1, c.argmax(dim=1, keepdim=True), stuck.unsqueeze(1))
    accept = accept | forced
    return torch.where(accept, proposal, blocks), int(accept.any(dim=1).sum())


def test_commit_tokens_hand_computed(device):
    M = 9
    blocks = torch.tensor([[M, M, 5, M],        # one above the threshold
                           [M, M, M, 7],        # none above: the most confident masked position is forced
                           [1, 2, 3, 4],        # nothing masked
                           [M, M, 6, M],        # the most confident proposal is the mask token itself: skipped
                           [M, M, M, M]], device=device)      # every proposal is the mask token: nothing to commit
    proposal = torch.tensor([[11, 12, 13, 14], [21, 22, 23, 24], [31, 32, 33, 34], [M, 42, 43, 44], [M, M, M, M]],
                            device=device)
    conf = torch.tensor([[0.2, 0.95, 0.99, 0.5], [0.3, 0.6, 0.6, 0.99], [0.9, 0.9, 0.9, 0.9], [0.99, 0.1, 0.99, 0.4],
                         [0.9, 0.9, 0.9, 0.9]], device=device)
    counter = torch.zeros(1, dtype=torch.int32, device=device)
    out = blocks.clone()
    ops.commit_tokens(out, proposal, conf, counter, M, 0.9)
    assert out.tolist() == [[M, 12, 5, M], [M, 22, M, 7], [1, 2, 3, 4], [M, M, 6, 44], [M, M, M, M]]
    assert counter.item() == 3
    ops.commit_tokens(out, proposal, conf, counter, M, 0.9)   # the counter accumulates; rows 0, 1 and 3 go on
    assert out.tolist() == [[M, 12, 5, 14], [M, 22, 23, 7], [1, 2, 3, 4], [M, 42, 6, 44], [M, M, M, M]]
    assert counter.item() == 6


@pytest.mark.parametrize("n,L", [(1, 1), (3, 4), (16, 32), (5, 64), (7, 100), (2, 300)])
def test_commit_tokens_equals_the_tensor_formulation(device, n, L):
    g = torch.Generator(device=device).manual_seed(n * 1000 + L)
    M = 63
    for trial in range(6):
        blocks = torch.randint(0, 63, (n, L), generator=g, device=device)
        blocks[torch.rand(n, L, generator=g, device=device) < (0.15 * trial)] = M
        proposal = torch.randint(0, 64, (n, L), generator=g, device=device)       # some proposals are the mask token
        conf = torch.rand(n, L, generator=g, device=device)
        conf = (conf * 8).round() / 8                                           # plenty of ties, also at the maximum
        threshold = [0.0, 0.5, 0.875, 1.0, 1.5, 0.9][trial]
        want, rows = _commit_rule(blocks, proposal, conf, M, threshold)
        counter = torch.zeros(1, dtype=torch.int32, device=device)
        got = blocks.clone()
        ops.commit_tokens(got, proposal, conf, counter, M, threshold)
        assert torch.equal(got, want) and counter.item() == rows
