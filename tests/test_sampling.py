"""Nucleus sampling of the generation loop (gpu/sample_utils.py:9-33 of the
reference): which tokens stay in the draw, and with which odds."""
import torch

from bitnet_amd.decoder import top_p_sample


def test_kept_set_is_the_shortest_prefix_whose_mass_exceeds_p():
    g = torch.Generator().manual_seed(0)
    # masses in front of the ranked tokens: 0, 0.5, 0.8, 0.95 -> with p = 0.7 the first two stay
    probs = torch.tensor([[0.15, 0.5, 0.05, 0.3]]).repeat(20000, 1)
    draws = top_p_sample(probs, 0.7, g).view(-1)
    counts = torch.bincount(draws, minlength=4).tolist()
    assert counts[0] == 0 and counts[2] == 0
    assert abs(counts[1] / 20000 - 0.625) < 0.015 and abs(counts[3] / 20000 - 0.375) < 0.015  # 0.5 : 0.3, renormalised
    # a mass of exactly p in front of a token keeps it (the comparison is strict)
    probs = torch.tensor([[0.5, 0.25, 0.25]]).repeat(4000, 1)
    counts = torch.bincount(top_p_sample(probs, 0.5, g).view(-1), minlength=3).tolist()
    assert counts[0] > 0 and counts[1] > 0 and counts[2] == 0


def test_tiny_p_is_greedy_and_rows_are_independent():
    g = torch.Generator().manual_seed(1)
    probs = torch.softmax(torch.randn(64, 300, generator=g), dim=-1)
    out = top_p_sample(probs, 1e-9, g)
    assert out.shape == (64, 1) and out.dtype == torch.int64
    assert torch.equal(out.view(-1), probs.argmax(dim=-1))
    # p = 1 keeps everything with non-zero probability
    probs = torch.tensor([[0.0, 1.0, 0.0], [0.0, 0.0, 1.0]])
    assert top_p_sample(probs, 1.0, g).view(-1).tolist() == [1, 2]


def test_same_generator_state_gives_the_same_draws():
    probs = torch.softmax(torch.randn(8, 50, generator=torch.Generator().manual_seed(2)), dim=-1)
    a = top_p_sample(probs, 0.9, torch.Generator().manual_seed(7))
    b = top_p_sample(probs, 0.9, torch.Generator().manual_seed(7))
    assert torch.equal(a, b)
