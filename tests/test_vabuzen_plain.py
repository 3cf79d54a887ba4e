"""The plain Vabuzen implementation by itself: what distinguishes the design's mechanisms moves its results by
far more than any tolerance the engine is held to (the one in the softmax's denominator, the pairing of the
rotation, the order of the taps, a window or a number of kept keys that is one off, the groups of experts, the
renormalization, the factor and the shared expert), and a row never depends on later tokens.  No GPU."""
import torch

import plain_vabuzen as plain
from helpers import random_tokens
from test_gpu_vabuzen import V1, attention_case, doubles, experts_case


def test_the_one_in_the_denominator_the_pairing_and_the_taps_show():
    """The plain attention with an ordinary softmax, with the halves paired instead of neighbours, with
    the taps in reverse order or with a window or a number of kept keys that is one off differs by far
    more than any tolerance."""
    t, m, _ = attention_case(60, 24, 2, 1, 16, 16, 0.5, 3, (100.0, 16), (9, 3))
    Wd = doubles(t)
    right = plain.window_attention(Wd["table"], Wd, "", m)

    def moved(out):
        return float((out - right).abs().max()) / float(right.abs().max())
    n = 60
    H, D = 2, 16
    # an ordinary softmax: the same scores, weights that sum to one
    q, k, v = (plain.causal_taps(Wd["table"] @ Wd[c].T, Wd[c + ".conv"]) for c in "qkv")
    pos = torch.arange(n)
    qh, kh = plain.rotate_neighbours(q.view(n, H, D), pos, 100.0, 16), plain.rotate_neighbours(k.view(n, 1, D), pos, 100.0, 16)
    out = torch.zeros(n, H, D, dtype=torch.float64)
    for i in range(n):
        seen = [j for j in range(i + 1) if i - j < 9 or j < 3]
        for a in range(H):
            out[i, a] = torch.softmax((kh[seen, 0] @ qh[i, a]) * 0.5, 0) @ v.view(n, 1, D)[seen, 0]
    assert moved(out.reshape(n, H * D) @ Wd["o"].T) > 0.1
    flipped = dict(Wd, **{c + ".conv": Wd[c + ".conv"].flip(1) for c in "qkv"})
    assert moved(plain.window_attention(Wd["table"], flipped, "", m)) > 0.1
    for size, keep in ((8, 3), (10, 3), (9, 2), (9, 4)):
        assert moved(plain.window_attention(Wd["table"], Wd, "", dict(m, mask={"size": size, "keep_first": keep}))) > 0.02, (size, keep)
    halves = plain.rotate_halves(q.view(n, H, D), pos, 100.0, 16)
    assert float((halves - qh).abs().max()) > 0.1 * float(qh.abs().max())


def test_the_groups_the_renormalization_and_the_shared_expert_show():
    """Without the groups other experts are chosen for many rows (the largest scores of a row often lie in a
    group that loses); weights not divided by their sum, a factor left out or the shared expert left out move
    the output by tens of percent."""
    t, f, _ = experts_case(64, 40, 24, 12, 3, (4, 2), 2.0, 40)
    Wd = doubles(t)
    right = plain.routed_ff(Wd["table"], Wd, "", f)
    score = torch.sigmoid(Wd["table"] @ Wd["router"].T)
    differ = sum(sorted(plain.choose_experts(score[i], f["router"])[0]) != sorted(plain.choose_experts(score[i], {"experts": 12, "top": 3})[0])
                 for i in range(64))
    assert differ >= 16
    moved = lambda out: float((out - right).abs().max()) / float(right.abs().max())
    assert moved(plain.routed_ff(Wd["table"], Wd, "", dict(f, router=dict(f["router"], scale=1.0)))) > 0.1
    assert moved(plain.routed_ff(Wd["table"], Wd, "", dict(f, shared=None))) > 0.1
    assert moved(plain.routed_ff(Wd["table"], Wd, "", dict(f, router=dict(f["router"], groups={"count": 4, "keep": 1})))) > 0.1


def test_a_row_does_not_depend_on_later_tokens(tmp_path):
    """Whole model, random weights: the logits of a prompt's first rows are those of the shorter prompt."""
    from test_gpu_vabuzen import write_model
    folder = write_model(tmp_path / "m", V1, 3)
    cfg, W = plain.load_model_folder(folder)
    toks = random_tokens(V1["vocab"], 50, seed=1)
    whole, part = plain.model_logits(cfg, W, toks), plain.model_logits(cfg, W, toks[:31])
    assert float((whole[:31] - part).abs().max()) <= 1e-6 * float(whole.abs().max())
    assert plain.greedy(cfg, W, toks[:5], 3) == plain.greedy(cfg, W, toks[:5], 4)[:3]
