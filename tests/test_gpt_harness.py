"""CPU checks of the minimal GPT used by the full-model parity case (tests/gpt_harness.py), with the oracle FFN.

These pin the harness itself, so that the GPU comparison (HIP FFN against oracle FFN inside the same model) means
something: the causal mask, the rotary embedding's relative-position property (the property the reference checks in
tests/test_rotary.py), the loss shift, the tied head and the padding row."""
import math

import torch

from gpt_harness import GPTConfig, MiniLeanGPT, apply_rotary, copy_parameters, rotary_tables

TINY = GPTConfig(vocab_size=97, embedding_size=48, hidden_size=32, num_layers=2, num_heads=4, intermediate_size=64,
                 layer_norm_eps=1e-5)


def test_loss_at_init_is_near_uniform():
    model = MiniLeanGPT(TINY, "oracle")
    ids = torch.randint(1, TINY.vocab_size, (3, 16), generator=torch.Generator().manual_seed(0))
    loss, logits = model(ids, labels=ids)
    assert logits.shape == (3, 16, TINY.vocab_size)
    assert abs(loss.item() - math.log(TINY.vocab_size)) < 0.5


def test_causal():
    """changing token t leaves the logits of positions < t unchanged"""
    model = MiniLeanGPT(TINY, "oracle").eval()
    ids = torch.randint(1, TINY.vocab_size, (2, 12), generator=torch.Generator().manual_seed(1))
    other = ids.clone()
    other[:, 7] = (other[:, 7] + 5) % (TINY.vocab_size - 1) + 1
    with torch.no_grad():
        a, b = model(ids), model(other)
    assert torch.allclose(a[:, :7], b[:, :7], atol=1e-5)
    assert not torch.allclose(a[:, 7:], b[:, 7:], atol=1e-5)


def test_rotary_is_relative():
    """<rot(q, i), rot(k, j)> depends on i - j only"""
    dim, seq = 16, 24
    cos, sin = rotary_tables(seq, dim, 10000, "cpu")
    gen = torch.Generator().manual_seed(2)
    q, k = torch.randn(dim, generator=gen), torch.randn(dim, generator=gen)
    rq = apply_rotary(q.expand(1, seq, 1, dim), cos, sin)[0, :, 0]
    rk = apply_rotary(k.expand(1, seq, 1, dim), cos, sin)[0, :, 0]
    dots = rq @ rk.t()
    for shift in (0, 3, 7):
        diag = torch.diagonal(dots, offset=-shift)
        assert torch.allclose(diag, diag[0].expand_as(diag), atol=1e-4)
    assert torch.allclose(rq.norm(dim=-1), q.norm().expand(seq), atol=1e-5)


def test_loss_shift_and_tied_head():
    model = MiniLeanGPT(TINY, "oracle")
    ids = torch.randint(1, TINY.vocab_size, (2, 10), generator=torch.Generator().manual_seed(3))
    loss, logits = model(ids, labels=ids)
    manual = torch.nn.functional.cross_entropy(logits[:, :-1].reshape(-1, TINY.vocab_size), ids[:, 1:].reshape(-1))
    assert torch.allclose(loss, manual, atol=1e-6)
    loss.backward()
    grad = model.word_embeddings.weight.grad
    assert grad is not None and grad[TINY.pad_token_id].abs().sum() > 0  # the tied head reaches the padding row too
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


def test_state_dict_carries_over():
    a, b = MiniLeanGPT(TINY, "oracle"), MiniLeanGPT(TINY, "oracle")
    b.reset_parameters(seed=5)
    copy_parameters(a, b)
    ids = torch.randint(1, TINY.vocab_size, (1, 8), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        assert torch.equal(a(ids), b(ids))
