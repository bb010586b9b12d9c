"""The probe model (tests/probe_model.py) does what it is for: its logits are
the weights of the visible keys by token, and the faults it exists to show — a
window off by one, one far key dropped, two pages of keys swapped — move a logit
by several times the bar the GPU tests use for it (no GPU)."""
import math
import random

import pytest
import torch

import plain_qwen2 as plain
import probe_model as pm
from replay_harness import probe_score


@pytest.fixture(scope="module")
def probe(tmp_path_factory):
    folder = pm.write_probe_model(str(tmp_path_factory.mktemp("probe")))
    return plain.load_folder(folder)


def tokens(n, seed):
    rng = random.Random(seed)
    return [rng.randrange(pm.PROBE["vocab_size"]) for _ in range(n)]


def test_logits_are_the_weights_of_the_visible_keys(probe):
    cfg, w = probe
    toks = tokens(90, 3)
    logits = plain.forward(cfg, w, toks)
    p = len(toks) - 1
    # layer 0, heads of a group prefer opposite signs: weight of key r is
    # exp(g u_r) / sum exp(g u) + exp(-g u_r) / sum exp(-g u)
    u = torch.tensor([pm.token_sign(t) for t in toks])
    weight = torch.softmax(pm.GAMMA * u, 0) + torch.softmax(-pm.GAMMA * u, 0)
    want = torch.zeros(pm.CODES)
    for r, t in enumerate(toks):
        want[t % pm.CODES] += weight[r]
    got = logits[p, :pm.CODES]
    assert torch.allclose(got / got.sum(), want / want.sum(), atol=2e-3)
    # layer 1 sees the last 24 keys only
    seen = {t % pm.CODES for t in toks[-24:]}
    window_logits = logits[p, pm.CODES:2 * pm.CODES]
    assert {i for i in range(pm.CODES) if window_logits[i] > 1e-3} == seen
    assert float(logits[p, 2 * pm.CODES:].abs().max()) == 0.0


@pytest.mark.parametrize("n,seed", [(200, 0), (600, 1)])
def test_faults_show_many_times_over_the_bar(probe, monkeypatch, n, seed):
    cfg, w = probe
    toks = tokens(n, seed)
    ref = plain.forward(cfg, w, toks)
    real = plain.visibility_mask

    def with_mask(mask):
        monkeypatch.setattr(plain, "visibility_mask", mask)
        try:
            return plain.forward(cfg, w, toks)
        finally:
            monkeypatch.setattr(plain, "visibility_mask", real)

    wider = with_mask(lambda q, k, window=None: real(q, k, None if window is None else window + 1))
    narrower = with_mask(lambda q, k, window=None: real(q, k, None if window is None else window - 1))
    for r in range(30, n):                             # every position past the first window shows it
        assert probe_score(wider[r], ref[r]) > 5 and probe_score(narrower[r], ref[r]) > 5

    def drop_first_key(q, k, window=None):
        vis = real(q, k, window).clone()
        if window is None:
            vis[-1, 0] = False                         # the farthest key of the last position
        return vis
    dropped = with_mask(drop_first_key)
    assert probe_score(dropped[-1], ref[-1]) > 5

    # two pages of 16 keys trade places in the K cache (V stays): the weights follow the wrong signs
    a, b = list(range(16, 32)), list(range(48, 64))
    real_rope = plain.apply_rope

    def swapped_keys(x, positions, inv_freq):
        y = real_rope(x, positions, inv_freq)
        if x.shape[1] == cfg["num_key_value_heads"]:
            y = y.clone()
            y[a + b] = y[b + a]
        return y
    monkeypatch.setattr(plain, "apply_rope", swapped_keys)
    swapped = plain.forward(cfg, w, toks)
    monkeypatch.setattr(plain, "apply_rope", real_rope)
    assert probe_score(swapped[-1], ref[-1]) > 5
