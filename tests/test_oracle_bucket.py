"""Pins oracle.relative_position_bucket (restates reference att.py:78-124).

Checks: a known-answer table computed from the closed form in exact arithmetic,
the installed HuggingFace implementation (third-party library), and brute force
over a distance range with python floats.
"""
import math

import pytest
import torch

from oracle import t5_basic as O

BI_FIRST = [8, 12, 16, 23, 32, 46, 64, 91]            # first distance of buckets 8..15 (32 buckets, max 128)
UNI_FIRST = [16, 19, 21, 24, 27, 31, 35, 40, 46, 52, 59, 67, 77, 87, 99, 113]  # first distance of buckets 16..31


def exact_bucket(rel, bidirectional, nb, md):
    """Closed form in python doubles with an integer-boundary guard (independent of torch's fp32 log)."""
    out = 0
    if bidirectional:
        nb //= 2
        if rel > 0:
            out += nb
        d = abs(rel)
    else:
        d = max(-rel, 0)
    me = nb // 2
    if d < me:
        return out + d
    x = math.log(d / me) / math.log(md / me) * (nb - me)
    r = round(x)
    if abs(x - r) < 1e-9:      # exact power: real arithmetic gives an integer
        x = r
    return out + min(me + int(x), nb - 1)


def test_known_answers_bidirectional():
    d = torch.arange(0, 300)
    b = O.relative_position_bucket(-d, True, 32, 128)       # key before query
    assert b[:8].tolist() == list(range(8))
    for k, first in enumerate(BI_FIRST):
        assert b[first].item() == 8 + k
        assert b[first - 1].item() == 8 + k - 1 if first > 8 else True
    assert (b[91:] == 15).all()
    after = O.relative_position_bucket(torch.tensor([1, 5, 8, 16, 127, 128, 5000]), True, 32, 128)
    assert after.tolist() == [17, 21, 24, 26, 31, 31, 31]
    assert O.relative_position_bucket(torch.tensor([0]), True, 32, 128).item() == 0


def test_known_answers_unidirectional():
    d = torch.arange(0, 300)
    b = O.relative_position_bucket(-d, False, 32, 128)
    assert b[:16].tolist() == list(range(16))
    for k, first in enumerate(UNI_FIRST):
        assert b[first].item() == 16 + k
        if first > 16:
            assert b[first - 1].item() == 16 + k - 1
    assert (b[113:] == 31).all()
    # future keys collapse to bucket 0
    assert (O.relative_position_bucket(torch.arange(1, 50), False, 32, 128) == 0).all()


@pytest.mark.parametrize("bidirectional", [True, False])
@pytest.mark.parametrize("nb,md", [(32, 128), (32, 64), (64, 256), (16, 128), (8, 32), (128, 1024)])
def test_against_exact_closed_form(bidirectional, nb, md):
    rel = torch.arange(-1300, 1301)
    got = O.relative_position_bucket(rel, bidirectional, nb, md).tolist()
    want = [exact_bucket(int(r), bidirectional, nb, md) for r in rel.tolist()]
    assert got == want


@pytest.mark.parametrize("bidirectional", [True, False])
@pytest.mark.parametrize("nb,md", [(32, 128), (64, 256), (20, 100)])
def test_against_huggingface(bidirectional, nb, md):
    from transformers.models.t5.modeling_t5 import T5Attention as HFT5Attention
    rel = torch.arange(-700, 701)[None, :] - torch.arange(0, 3)[:, None]
    want = HFT5Attention._relative_position_bucket(rel, bidirectional=bidirectional, num_buckets=nb, max_distance=md)
    got = O.relative_position_bucket(rel, bidirectional, nb, md)
    assert torch.equal(got, want)


def test_compute_bias_is_gather_of_buckets():
    table = torch.randn(32, 5)
    bias = O.compute_bias(table, 7, 300, True)
    assert bias.shape == (1, 5, 7, 300)
    for (i, j) in [(0, 0), (3, 200), (6, 1), (2, 2), (5, 299)]:
        b = exact_bucket(j - i, True, 32, 128)
        assert torch.equal(bias[0, :, i, j], table[b])
