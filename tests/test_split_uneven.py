"""``split_tensor_uneven`` / ``remove_padding_after_gather`` against the rule of the reference
(utils.py:86-136 and :142-167): shard i of ``world_size`` gets ``S // N`` tokens, the first ``S % N``
shards one more; every shard is zero-padded at its END to ``ceil(S / N)`` tokens; the pad sizes are
filed under the tensor's name and ``remove_padding_after_gather`` drops exactly those rows from the
concatenation of the shards along dim 1.

The expectations below are written out from that rule (lengths, pad positions, values), not computed by
calling the function under test a second time.
"""
import pytest
import torch

from ditango_amd import utils


@pytest.fixture(autouse=True)
def _fresh_padding_dict():
    utils.get_padding_dict().clear()
    yield
    utils.get_padding_dict().clear()


def _expected_lengths(S, N):
    return [S // N + (1 if i < S % N else 0) for i in range(N)]


@pytest.mark.parametrize("S,N", [(10, 4), (17776, 8), (119056, 32), (7, 8), (16, 4), (5, 1), (9, 2)])
def test_shard_lengths_pads_and_values_dim1(S, N):
    x = torch.arange(1, 2 * S * 3 + 1, dtype=torch.float32).view(2, S, 3)       # no zeros among the real rows
    parts = utils.split_tensor_uneven(x, N, dim=1, tensor_name="x")
    lens = _expected_lengths(S, N)
    target = -(-S // N)
    assert len(parts) == N and sum(lens) == S
    assert utils.get_padding_dict()["x"] == [target - n for n in lens]
    start = 0
    for i, part in enumerate(parts):
        assert tuple(part.shape) == (2, target, 3) and part.dtype == x.dtype
        assert torch.equal(part[:, :lens[i]], x[:, start:start + lens[i]])          # real rows first, in order
        assert torch.count_nonzero(part[:, lens[i]:]) == 0                           # zero rows behind them
        start += lens[i]
    if S % N == 0:
        assert utils.get_padding_dict()["x"] == [0] * N
    else:
        # the first S % N shards are full, every later one carries exactly one padded row
        assert utils.get_padding_dict()["x"] == [0] * (S % N) + [1] * (N - S % N)


def test_split_along_dim0_and_without_a_name():
    x = torch.arange(1, 11 * 2 + 1, dtype=torch.bfloat16).view(11, 2)
    parts = utils.split_tensor_uneven(x, 4, dim=0)                                   # 3, 3, 3, 2 (+1 zero row)
    assert [tuple(p.shape) for p in parts] == [(3, 2)] * 4
    assert torch.equal(parts[0], x[0:3]) and torch.equal(parts[2], x[6:9])
    assert torch.equal(parts[3][:2], x[9:11]) and torch.count_nonzero(parts[3][2:]) == 0
    assert utils.get_padding_dict() == {}                                            # no name, no book-keeping


@pytest.mark.parametrize("S,N", [(10, 4), (2222 * 8 - 3, 8), (7, 8), (12, 3)])
def test_round_trip_through_a_gather(S, N):
    """Shards concatenated along dim 1 (what the all-gather of the callers produces), padding removed:
    the original tensor, bit for bit."""
    x = torch.randn(2, S, 4, generator=torch.Generator().manual_seed(S * N))
    parts = utils.split_tensor_uneven(x, N, dim=1, tensor_name="hidden")
    gathered = torch.cat(parts, dim=1)
    assert gathered.shape[1] == N * -(-S // N)
    back = utils.remove_padding_after_gather(gathered, "hidden")
    assert torch.equal(back, x)


def test_remove_padding_is_the_identity_for_unknown_names_and_keeps_names_apart():
    x = torch.randn(1, 10, 2)
    y = torch.randn(1, 9, 2)
    px = utils.split_tensor_uneven(x, 4, tensor_name="x")       # pads 0 0 1 1
    py = utils.split_tensor_uneven(y, 2, tensor_name="y")       # pads 0 1
    assert utils.get_padding_dict() == {"x": [0, 0, 1, 1], "y": [0, 1]}
    gx, gy = torch.cat(px, dim=1), torch.cat(py, dim=1)
    assert utils.remove_padding_after_gather(gx, "never split") is gx
    assert torch.equal(utils.remove_padding_after_gather(gx, "x"), x)
    assert torch.equal(utils.remove_padding_after_gather(gy, "y"), y)
    # a later split under the same name replaces the entry (utils.py:133-134)
    utils.split_tensor_uneven(torch.randn(1, 8, 2), 4, tensor_name="x")
    assert utils.get_padding_dict()["x"] == [0, 0, 0, 0]


def test_padded_rows_take_part_in_the_oracle_softmax_with_score_zero():
    """What the zero rows do downstream (the dense path does not mask them, utils.py:120-127): a zero key
    has score 0 against every query and a zero value adds nothing to the numerator, so one padded key
    raises exp(lse) by exactly 1 and scales out by sum / (sum + 1)."""
    from oracle import attention_math as om
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 5, 2, 16, generator=g) for _ in range(3))
    o0, l0 = om.chunk_attention(q, k, v)
    kp = torch.cat([k, torch.zeros(1, 1, 2, 16)], dim=1)
    vp = torch.cat([v, torch.zeros(1, 1, 2, 16)], dim=1)
    o1, l1 = om.chunk_attention(q, kp, vp)
    z0 = l0.double().exp()
    assert torch.allclose(l1.double().exp(), z0 + 1.0, rtol=1e-5)
    w = (z0 / (z0 + 1.0)).transpose(1, 2).unsqueeze(-1)                              # [B,H,S] -> [B,S,H,1]
    assert torch.allclose(o1.double(), o0.double() * w, atol=1e-5)
