"""What pins the plain implementation beside the reference's text: the reference's own test
vectors, special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a tap order)
fails it."""
import math

import numpy as np
import pytest
import scipy.signal
import scipy.special

from plain import lfm2 as P
from plain import sampler as S
from tiny import write_tiny

RNG = np.random.default_rng(0)


# -- RMSNorm --------------------------------------------------------------------------------
def test_rmsnorm():
    x = RNG.normal(size=(5, 96)) * 3
    w = 1 + 0.15 * RNG.normal(size=96)
    y = P.rmsnorm(x, w, 1e-5)
    assert np.allclose(y, x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-5) * w)
    assert np.allclose(np.sqrt((P.rmsnorm(x, np.ones(96), 0.0) ** 2).mean(-1)), 1.0)  # unit RMS
    assert np.allclose(P.rmsnorm(7.0 * x, w, 0.0), P.rmsnorm(x, w, 0.0))              # scale free
    z = P.rmsnorm(np.zeros((1, 8)), np.ones(8), 1e-5)
    assert np.isfinite(z).all() and not z.any()         # eps inside the root: 0 stays 0, finite
    # eps outside the root would give 1/(1+eps), not 1/sqrt(1+eps)
    one = P.rmsnorm(np.ones((1, 4)), np.ones(4), 3.0)
    assert np.allclose(one, 0.5)
    # the weight multiplies after the normalisation, it is not part of the mean
    assert np.allclose(P.rmsnorm(x, 2 * w, 1e-5), 2 * P.rmsnorm(x, w, 1e-5))


def test_per_head_norm_shares_one_weight():
    x = RNG.normal(size=(3, 4, 16))
    w = 1 + 0.1 * RNG.normal(size=16)
    y = P.per_head_rmsnorm(x, w, 1e-6)
    for h in range(4):
        assert np.allclose(y[:, h], P.rmsnorm(x[:, h], w, 1e-6))
    x2 = x.copy()
    x2[:, 1] *= 100                                      # heads are independent
    assert np.allclose(P.per_head_rmsnorm(x2, w, 1e-6)[:, [0, 2, 3]], y[:, [0, 2, 3]])


# -- rotation --------------------------------------------------------------------------------
def test_rope_pairs_and_sign():
    d = 16
    e0 = np.zeros((1, 1, d))
    e0[0, 0, 0] = 1.0
    y = P.rope_neox(e0, [1], 10000.0)
    # index 0 pairs with index d/2 (not with 1), and turns towards +sin
    assert np.isclose(y[0, 0, 0], math.cos(1.0)) and np.isclose(y[0, 0, d // 2], math.sin(1.0))
    assert np.allclose(np.delete(y[0, 0], [0, d // 2]), 0)
    x = RNG.normal(size=(6, 3, d))
    assert np.allclose(P.rope_neox(x, [0] * 6, 1e6), x)                      # position 0
    y = P.rope_neox(x, np.arange(6), 1e6)
    assert np.allclose((y ** 2).sum(-1), (x ** 2).sum(-1))                   # a rotation
    # as a complex multiplication on (x_j + i x_{j+d/2})
    ang = P.rope_angles(np.arange(6), d, 1e6)
    z = (x[..., :d // 2] + 1j * x[..., d // 2:]) * np.exp(1j * ang)[:, None, :]
    assert np.allclose(y, np.concatenate([z.real, z.imag], -1))
    # frequencies: theta^(-2j/d); the last pair turns slowest
    assert np.allclose(ang[1], 1e6 ** (-2 * np.arange(d // 2) / d))


def test_rope_scores_depend_on_distance_only():
    d = 32
    q, k = RNG.normal(size=(1, 1, d)), RNG.normal(size=(1, 1, d))
    def score(pq, pk):
        return float((P.rope_neox(q, [pq], 1e4) * P.rope_neox(k, [pk], 1e4)).sum())
    assert np.isclose(score(5, 2), score(105, 102)) and np.isclose(score(9, 9), score(0, 0))
    assert not np.isclose(score(5, 2), score(2, 5))


# -- attention --------------------------------------------------------------------------------
def test_attention_reduces_to_library_softmax():
    T, H, d = 7, 3, 8
    q, k, v = (RNG.normal(size=(T, H, d)) for _ in range(3))
    out = P.causal_attention(q, k, v)                  # G = H: plain multi-head attention
    for h in range(H):
        sc = q[:, h] @ k[:, h].T / math.sqrt(d)
        sc[np.triu_indices(T, 1)] = -np.inf
        assert np.allclose(out[:, h], scipy.special.softmax(sc, axis=-1) @ v[:, h])


def test_attention_special_cases():
    T, H, G, d = 6, 4, 2, 8
    q = RNG.normal(size=(T, H, d))
    k, v = RNG.normal(size=(T, G, d)), RNG.normal(size=(T, G, d))
    out = P.causal_attention(q, k, v)
    assert np.allclose(out[0], np.repeat(v[0], H // G, axis=0))        # one key: its value
    # heads 0,1 read kv head 0 and heads 2,3 read kv head 1
    k2, v2 = k.copy(), v.copy()
    k2[:, 1] += 5
    v2[:, 1] -= 3
    out2 = P.causal_attention(q, k2, v2)
    assert np.allclose(out2[:, :2], out[:, :2]) and not np.allclose(out2[:, 2:], out[:, 2:])
    # equal keys: the mean of the values seen so far
    ke = np.broadcast_to(k[:1], k.shape)
    oe = P.causal_attention(q, ke, v)
    assert np.allclose(oe[3, 0], v[:4, 0].mean(0))
    # a row does not see later tokens
    k3, v3 = k.copy(), v.copy()
    k3[4:] = 9
    v3[4:] = -9
    assert np.allclose(P.causal_attention(q, k3, v3)[:4], out[:4])
    # a window of 3 keeps the last three keys, the row's own included
    ow = P.causal_attention(q, k, v, window=3)
    assert np.allclose(ow[:3], out[:3])
    assert np.allclose(ow[5], P.causal_attention(q[3:], k[3:], v[3:])[2])


# -- short convolution ------------------------------------------------------------------------
def test_conv_is_a_causal_fir_filter():
    T, D, L = 11, 5, 4
    bx, w = RNG.normal(size=(T, D)), RNG.normal(size=(D, L))
    s = P.causal_short_conv(bx, w)
    for c in range(D):
        assert np.allclose(s[:, c], scipy.signal.lfilter(w[c, ::-1], [1.0], bx[:, c]))
        assert np.allclose(s[:, c], np.convolve(bx[:, c], w[c, ::-1])[:T])
    ident = np.zeros((D, L))
    ident[:, -1] = 1.0                                 # the last tap meets the current token
    assert np.allclose(P.causal_short_conv(bx, ident), bx)
    delay = np.zeros((D, L))
    delay[:, 0] = 1.0                                  # the first tap meets the oldest
    assert np.allclose(P.causal_short_conv(bx, delay)[L - 1:], bx[:T - L + 1])
    assert np.allclose(P.causal_short_conv(bx, w, np.ones(D)), s + 1)


def test_conv_against_the_reference_tests_second_formulation():
    """Inputs and the expectation loop of src/test/test_hybrid.c:78-151 (stateful causal part),
    with the state written as zeros before the sequence: the plain whole-sequence function
    must give what that loop gives when its initial state is zero, and, run on a sequence
    with a prefix, what the loop gives from the state that the prefix leaves."""
    for dim in (1, 3, 4, 7, 16, 33):
        for n in (1, 2, 9):
            for kernel in (2, 3, 4):
                hist = kernel - 1
                in_stride = 3 * dim + 3
                mixed = np.array([((i % 23) - 11) / 17.0 for i in range((n + hist) * in_stride)],
                                 dtype=np.float64).reshape(n + hist, in_stride)
                weights = np.array([((i % 17) - 8) / 19.0 for i in range(dim * kernel)]).reshape(
                    dim, kernel)
                Bq, Cq, Xq = mixed[:, :dim], mixed[:, dim:2 * dim], mixed[:, 2 * dim:3 * dim]
                bx = Bq * Xq
                # the reference's loop on the last n rows, its state = bx of the hist rows before
                initial = bx[:hist].T                   # [dim, hist], oldest first
                expect = np.zeros((n, dim))
                for t in range(n):
                    for c in range(dim):
                        total = 0.0
                        for k in range(kernel):
                            source = t + k - hist
                            b = initial[c, source + hist] if source < 0 else bx[hist + source, c]
                            total += b * weights[c, k]
                        expect[t, c] = Cq[hist + t, c] * total
                # hist zero rows in front make "before the sequence" explicit
                pad = np.zeros((hist, dim))
                s = P.causal_short_conv(np.concatenate([pad, bx]), weights)[hist:]
                got = (Cq * s)[hist:]
                assert np.abs(got - expect).max() < 1e-12, (dim, n, kernel)


def test_conv_mixer_order_of_the_three_parts():
    cfg = {"hidden_size": 4}
    D = 4
    lw = {"in_proj": RNG.normal(size=(3 * D, D)), "conv": np.zeros((D, 3)),
          "out_proj": np.eye(D)}
    lw["conv"][:, -1] = 1.0
    xb = RNG.normal(size=(5, D))
    p = xb @ lw["in_proj"].T
    # B, C, x in this order: with identity taps the mixer gives C * (B * x)
    assert np.allclose(P.short_conv_mixer(xb, lw, cfg), p[:, D:2 * D] * p[:, :D] * p[:, 2 * D:])


def test_conv_mixer_biases_are_those_of_the_library_layers():
    """With ``conv_bias`` the checkpoint holds a bias for each of the three linear maps of the
    mixer: ``in_proj.bias``, ``conv.bias`` (the depthwise convolution's own, so it is added to the
    filter's output, before the C gate) and ``out_proj.bias``.  kappai's LFM2 has no biases, so
    this is pinned by the library routines that such tensors belong to: a linear layer with bias,
    a grouped 1-d convolution with bias and left padding, a linear layer with bias.  A bias added
    after the gate, or to the gated input, fails."""
    import torch
    import torch.nn.functional as F
    D, L, T = 6, 4, 9
    cfg = {"hidden_size": D}
    lw = {"in_proj": RNG.normal(size=(3 * D, D)), "in_proj_bias": RNG.normal(size=3 * D),
          "conv": RNG.normal(size=(D, L)), "conv_bias": RNG.normal(size=D),
          "out_proj": RNG.normal(size=(D, D)), "out_proj_bias": RNG.normal(size=D)}
    xb = RNG.normal(size=(T, D))
    t = {k: torch.from_numpy(np.asarray(v)) for k, v in lw.items()}
    p = F.linear(torch.from_numpy(xb), t["in_proj"], t["in_proj_bias"])
    Bg, Cg, xg = p[:, :D], p[:, D:2 * D], p[:, 2 * D:]
    bx = (Bg * xg).T[None]                                   # [1, channels, time]
    s = F.conv1d(bx, t["conv"][:, None, :], t["conv_bias"], padding=L - 1, groups=D)[0, :, :T].T
    want = F.linear(Cg * s, t["out_proj"], t["out_proj_bias"]).numpy()
    got = P.short_conv_mixer(xb, lw, cfg)
    assert np.abs(got - want).max() < 1e-12
    # the plausible mistakes give something else
    late = F.linear(Cg * (s - t["conv_bias"]) + t["conv_bias"], t["out_proj"], t["out_proj_bias"]).numpy()
    assert np.abs(got - late).max() > 1e-3


# -- feed-forward, head --------------------------------------------------------------------------
def test_swiglu():
    xb = RNG.normal(size=(4, 8))
    lw = {"w1": RNG.normal(size=(12, 8)), "w3": RNG.normal(size=(12, 8)), "w2": RNG.normal(size=(8, 12))}
    g, u = xb @ lw["w1"].T, xb @ lw["w3"].T
    assert np.allclose(P.swiglu_feed_forward(xb, lw), (g / (1 + np.exp(-g)) * u) @ lw["w2"].T)
    assert P.silu(np.zeros(1))[0] == 0 and np.isclose(P.silu(np.array([50.0]))[0], 50.0)
    lw0 = dict(lw, w1=np.zeros((12, 8)))
    assert not P.swiglu_feed_forward(xb, lw0).any()      # the gate, not the up branch, is activated


def test_whole_model_invariants(tmp_path):
    d = write_tiny("A", tmp_path / "a")
    cfg, w = P.read_model_dir(d)
    toks = [3, 200, 17, 17, 0, 255, 9, 41, 41, 100]
    full = P.forward(cfg, w, toks)
    assert full.shape == (10, 256) and np.isfinite(full).all()
    # causal: a prefix gives the same logits
    assert np.allclose(P.forward(cfg, w, toks[:6]), full[:6], atol=1e-12)
    # with the mixers' and feed-forwards' output maps zeroed the model is head(norm(E[token]))
    w0 = dict(w)
    for k in w:
        if k.endswith("out_proj.weight") or k.endswith("w2.weight"):
            w0[k] = np.zeros_like(w[k])
    E = w["model.embed_tokens.weight"]
    x = E[toks]
    expect = P.rmsnorm(x, w["model.embedding_norm.weight"], cfg["norm_eps"]) @ E.T
    assert np.allclose(P.forward(cfg, w0, toks), expect)
    # tied: an untied copy of the table as head gives the same
    cfg_u = dict(cfg, tie_embedding=False)
    assert np.allclose(P.forward(cfg_u, dict(w, **{"lm_head.weight": E}), toks), full)
    # the mixers matter: zeroing one attention layer's output map changes later logits only
    w1 = dict(w)
    w1["model.layers.1.self_attn.out_proj.weight"] = np.zeros_like(w["model.layers.1.self_attn.out_proj.weight"])
    assert np.abs(P.forward(cfg, w1, toks) - full).max() > 1e-3


@pytest.mark.parametrize("name", ["A", "B", "C", "E", "F"])
def test_two_statements_of_the_whole_model_agree(tmp_path, name):
    """The whole-sequence statement (``plain/lfm2.py``: no state, masks and sums over the whole
    sequence) and the token-by-token statement (``plain/lfm2_steps.py``: a shift register per conv
    layer, keys and values appended per token, rotation as complex numbers), written apart from
    each other, give the same logits for every position.  A wrong tap order, a state that is
    shifted the wrong way, a rotation with the wrong sign or pairing, a norm on the wrong side of
    the rotation, or a head read from the wrong kv group would have to be wrong in both forms."""
    from plain import lfm2_steps
    d = write_tiny(name, tmp_path / name.lower())
    cfg, w = P.read_model_dir(d)
    rng = np.random.default_rng(31)
    toks = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=14)]
    whole = P.forward(cfg, w, toks)
    steps = lfm2_steps.forward_by_steps(cfg, w, toks)
    assert steps.shape == whole.shape
    assert np.abs(steps - whole).max() < 1e-10 * max(1.0, np.abs(whole).max())


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_logits_of_some_rows_only(tmp_path, name):
    """``forward(..., rows=...)`` works out, in the attention layers, only the rows that the
    wanted logits depend on (what long sequences need to stay affordable): the wanted rows equal
    those of the whole computation, the others are marked as not computed; the rows a
    layer must deliver follow the FIR's reach backwards and stop at an attention layer, which
    needs every row before it."""
    assert P.rows_needed(["conv", "attention", "conv"], 3, [9]) == [None, {7, 8, 9}, {9}]
    assert P.rows_needed(["attention", "conv", "conv"], 4, [1, 20]) == [
        {0, 1, 14, 15, 16, 17, 18, 19, 20}, {0, 1, 17, 18, 19, 20}, {1, 20}]
    assert P.rows_needed(["attention", "attention"], 3, [5]) == [None, {5}]
    d = write_tiny(name, tmp_path / name.lower())
    cfg, w = P.read_model_dir(d)
    rng = np.random.default_rng(32)
    toks = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=23)]
    whole = P.forward(cfg, w, toks)
    for rows in ([22], [0, 7, 21, 22], list(range(23))):
        some = P.forward(cfg, w, toks, rows=rows)
        # (not bit for bit: the head's product over fewer rows adds in another order)
        assert np.abs(some[rows] - whole[rows]).max() < 1e-12 * np.abs(whole).max()
        others = [r for r in range(23) if r not in rows]
        assert np.isnan(some[others]).all()


def test_conv_bias_and_untied_head_are_used(tmp_path):
    d = write_tiny("B", tmp_path / "b")
    cfg, w = P.read_model_dir(d)
    toks = list(range(20, 32))
    full = P.forward(cfg, w, toks)
    for name in ("model.layers.1.conv.in_proj.bias", "model.layers.1.conv.conv.bias",
                 "model.layers.1.conv.out_proj.bias", "lm_head.weight"):
        w2 = dict(w)
        w2[name] = w[name] + 0.5
        assert np.abs(P.forward(cfg, w2, toks) - full).max() > 1e-3, name


def test_round_bf16():
    x = np.array([1.0, 1.0 + 2 ** -9, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -9, -3.14159, 1e-30, 0.0])
    r = P.round_bf16(x)
    # ties go to the even mantissa: 1 + 2^-8 lies half way between 1 and 1 + 2^-7
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == 1.0 and r[3] == 1.0 + 2 ** -7
    import torch
    assert np.array_equal(r, torch.tensor(x, dtype=torch.float32).to(torch.bfloat16).double().numpy())


# -- sampler -----------------------------------------------------------------------------------
PROBS8 = np.array([0.5, 0.2, 0.15, 0.1, 0.03, 0.01, 0.007, 0.003], dtype=np.float32)


def draws(seed, logits, n=10000, **kw):
    s = S.PlainSampler(seed, repeat_penalty=1.0, **kw)
    return np.bincount([s.sample(logits) for _ in range(n)], minlength=len(logits))


def test_sampler_laws_of_the_reference_tests():
    """src/test/test_sampler.c:50-239 with its seeds and bounds."""
    lg = np.log(PROBS8)
    c = draws(42, lg, temperature=1.0, top_k=3, top_p=1.0, min_p=0.0)
    assert (c[3:] == 0).all() and c[0] > 4500 and c[1] > 1500 and c[2] > 1000
    c = draws(7, lg, temperature=1.0, top_k=0, top_p=0.71, min_p=0.0)
    assert (c[:3] > 0).all() and (c[3:] == 0).all()         # the crossing token is kept
    c = draws(7, lg, temperature=1.0, top_k=0, top_p=0.45, min_p=0.0)
    assert c[0] == 10000
    c = draws(99, lg, temperature=1.0, top_k=0, top_p=1.0, min_p=0.35)
    assert (c[:2] > 0).all() and (c[2:] == 0).all()
    c = draws(99, lg, temperature=1.0, top_k=0, top_p=1.0, min_p=0.21)
    assert (c[:3] > 0).all() and (c[3:] == 0).all()
    two = np.array([1.0, 0.0], dtype=np.float32)
    f = [draws(1234, two, temperature=t, top_k=0, top_p=1.0, min_p=0.0)[0] / 10000
         for t in (0.5, 1.0, 2.0)]
    assert 0.85 <= f[0] <= 0.91 and 0.70 <= f[1] <= 0.76 and 0.59 <= f[2] <= 0.65


def test_sampler_greedy_ties_seed_and_penalty():
    lg = np.array([0.1, 2.0, 2.0, -1.0], dtype=np.float32)
    assert S.PlainSampler(5, temperature=0.0).sample(lg) == 1           # lowest id on ties
    assert S.PlainSampler(5, temperature=1.0, top_k=1).sample(lg) == 1
    a = S.PlainSampler(77, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0)
    b = S.PlainSampler(77, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0)
    wide = RNG.normal(size=50).astype(np.float32)
    assert [a.sample(wide) for _ in range(50)] == [b.sample(wide) for _ in range(50)]
    s = S.PlainSampler(1, temperature=0.0, repeat_penalty=2.0)
    s.observe(0)
    assert s.sample(np.array([1.0, 0.9, 0.0, -1.0], dtype=np.float32)) == 1
    # the full-vocabulary path and the filtered path with nothing filtered agree in law
    lg8 = np.log(PROBS8)
    full = draws(3, lg8, n=4000, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0) / 4000
    filt = draws(3, lg8, n=4000, temperature=1.0, top_k=8 - 1, top_p=1.0, min_p=0.0) / 4000
    assert np.abs(full[:4] - PROBS8[:4]).max() < 0.03 and np.abs(filt[:4] - full[:4]).max() < 0.04


def test_rng_stream():
    r = S.Rng(0)
    assert r.s == S.Rng(0xDEADBEEFCAFEBABE).s           # seed 0 stands for this constant
    u = [S.Rng(9).uniform() for _ in range(3)]
    assert u[0] == u[1] == u[2] and 0.0 <= u[0] < 1.0
    xs = [r.uniform() for _ in range(2000)]
    assert 0.45 < np.mean(xs) < 0.55 and min(xs) >= 0 and max(xs) < 1
    assert all(float(x * 2 ** 24).is_integer() for x in xs[:50])
    # splitmix64 from state 0: the published first output of that generator
    assert S.splitmix64(0)[1] == 0xE220A8397B1DCDAF
