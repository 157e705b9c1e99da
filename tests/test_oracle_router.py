"""Pins of the router-gate oracle (CPU): against torch.topk where the answer is unique, closed
forms, a scalar brute-force loop, and a hand-worked group-limit case."""

import math

import pytest
import torch

from oracle import router as R


def _logits(T, E, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((T, E), generator=g) * 2).to(dtype)


@pytest.mark.parametrize("E,k", [(128, 8), (64, 6), (32, 4), (160, 6)])
def test_selected_sets_equal_torch_topk_without_ties(E, k):
    lg = _logits(200, E, E + k)  # fp32 normal draws: no two scores tie
    idx, w, scores = R.softmax_topk(lg, k)
    ref_w, ref_idx = torch.topk(lg.softmax(-1, dtype=torch.float32), k, dim=-1, sorted=True)
    assert torch.equal(idx, ref_idx) and torch.equal(w, ref_w)
    idx1, w1, _ = R.topk_softmax(lg, k)
    top_l, top_i = torch.topk(lg, k, dim=-1, sorted=True)
    assert torch.equal(idx1, top_i) and torch.equal(w1, torch.softmax(top_l, -1))


def test_closed_forms():
    # uniform logits: every score is 1/E, ties go to the lowest indices, renormalised weights 1/k
    lg = torch.full((3, 16), 0.7)
    idx, w, scores = R.softmax_topk(lg, 4, norm_topk_prob=True)
    assert torch.equal(idx, torch.arange(4).expand(3, 4))
    torch.testing.assert_close(scores, torch.full((3, 16), 1 / 16))
    torch.testing.assert_close(w, torch.full((3, 4), 0.25))
    idx, w, _ = R.topk_softmax(lg, 4)
    assert torch.equal(idx, torch.arange(4).expand(3, 4))
    torch.testing.assert_close(w, torch.full((3, 4), 0.25))
    # logits log(1), log(2), log(3), log(4): scores i/10; top-2 = experts 3, 2 with 0.4, 0.3
    lg = torch.log(torch.tensor([[1.0, 2.0, 3.0, 4.0]]))
    idx, w, scores = R.softmax_topk(lg, 2)
    assert idx.tolist() == [[3, 2]]
    torch.testing.assert_close(w, torch.tensor([[0.4, 0.3]]))
    idx, w, _ = R.softmax_topk(lg, 2, norm_topk_prob=True, scale=2.5)
    torch.testing.assert_close(w, torch.tensor([[4 / 7, 3 / 7]]) * 2.5)
    idx, w, _ = R.topk_softmax(lg, 2)  # softmax over log 4, log 3 = 4/7, 3/7
    assert idx.tolist() == [[3, 2]]
    torch.testing.assert_close(w, torch.tensor([[4 / 7, 3 / 7]]))


def test_scalar_brute_force():
    T, E, k = 6, 12, 3
    lg = _logits(T, E, 5)
    lg[2, 4] = lg[2, 9]  # an exact tie inside a row
    idx, w, scores = R.softmax_topk(lg, k, norm_topk_prob=True)
    for t in range(T):
        ex = [math.exp(float(lg[t, e]) - float(lg[t].max())) for e in range(E)]
        sc = [v / sum(ex) for v in ex]
        order = sorted(range(E), key=lambda e: (-float(scores[t, e]), e))[:k]  # by the fp32 scores, index breaks ties
        assert idx[t].tolist() == order
        tot = sum(sc[e] for e in order)
        for j, e in enumerate(order):
            assert abs(float(w[t, j]) - sc[e] / tot) < 1e-6
            assert abs(float(scores[t, e]) - sc[e]) < 1e-6


def test_group_limit_hand_worked():
    # 8 experts in 4 groups of 2; group maxima: g0 = 0.05, g1 = 0.40, g2 = 0.25, g3 = 0.10 (as scores)
    probs = torch.tensor([[0.05, 0.02, 0.40, 0.03, 0.25, 0.10, 0.10, 0.05]])
    lg = probs.log()
    idx, w, scores = R.softmax_topk(lg, 3, num_group=4, topk_group=2)
    # groups 1 and 2 stay: experts 2, 3, 4, 5; the best three are 2 (0.40), 4 (0.25), 5 (0.10)
    assert idx.tolist() == [[2, 4, 5]]
    torch.testing.assert_close(w, torch.tensor([[0.40, 0.25, 0.10]]))
    assert scores[0, [0, 1, 6, 7]].abs().max() == 0 and (scores[0, 2:6] > 0).all()
    # expert 6 (0.10) ties expert 5 but sits in a dropped group: never chosen, and no gradient reaches it
    l2 = lg.clone().requires_grad_(True)
    R.softmax_topk(l2, 3, num_group=4, topk_group=2)[1].sum().backward()
    full = lg.clone().requires_grad_(True)
    s = full.softmax(-1)
    (s[0, 2] + s[0, 4] + s[0, 5]).backward()
    torch.testing.assert_close(l2.grad, full.grad)


def test_weights_sum_and_forced_selection():
    lg = _logits(50, 64, 9, torch.bfloat16)
    _, w, _ = R.softmax_topk(lg, 6, norm_topk_prob=True, scale=16.0)
    torch.testing.assert_close(w.sum(-1), torch.full((50,), 16.0))
    _, w, _ = R.topk_softmax(lg, 4)
    torch.testing.assert_close(w.sum(-1), torch.ones(50))
    forced = torch.randint(0, 64, (50, 6), generator=torch.Generator().manual_seed(1))
    idx, w, scores = R.softmax_topk(lg, 6, forced_idx=forced)
    assert torch.equal(idx, forced) and torch.equal(w, scores.gather(-1, forced))
