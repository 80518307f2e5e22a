"""A second statement of the LFM2 forward pass: one token at a time with running state, the way
kappai decodes, written apart from ``lfm2.py`` (which states whole sequences without state).

It shares nothing with ``lfm2.py`` but the reader of the model folder: the norm is written with
an explicit loop-free sum and division, rotation as a multiplication of complex numbers, the
convolution as the shift register of ``shortconv_causal_chunk``, attention over lists of keys
and values that grow by one per token, the feed-forward with the logistic function spelled
out.  ``tests/test_plain.py`` holds the two against each other: a mistake would have to be made
twice, in two different forms, to pass.
"""
from __future__ import annotations

import cmath
import math

import numpy as np


def _norm(v, weight, eps):
    """src/backend/cpu/scalar/quants.c:1507-1512: sum of squares / n + eps under the root, the
    weight after the scaling."""
    n = v.shape[-1]
    scale = 1.0 / math.sqrt(float(np.dot(v, v)) / n + eps)
    return np.array([v[i] * scale * weight[i] for i in range(n)])


def _rotate(head, position, theta):
    """src/backend/cpu/quants.h:395-409 with the angles of src/compute.c:22-56: element j and
    element j + d/2 are the real and imaginary part of one number, turned by
    position * theta^(-2j/d)."""
    d = head.shape[0]
    half = d // 2
    out = np.empty(d)
    for j in range(half):
        z = complex(head[j], head[j + half]) * cmath.exp(1j * position * theta ** (-2.0 * j / d))
        out[j], out[j + half] = z.real, z.imag
    return out


class ConvState:
    """The shift register of one conv layer (src/backend/cpu/common.c:2393-2431): ``hist`` holds
    the last L-1 values of B*x, oldest first, zero before the sequence starts
    (src/recipe/ops_hybrid.c:353-354)."""

    def __init__(self, width, taps):
        self.hist = np.zeros((taps - 1, width))

    def step(self, b, c, x, w, bias):
        bx = b * x
        total = bx * w[:, -1]
        for k in range(self.hist.shape[0]):
            total = total + self.hist[k] * w[:, k]
        if bias is not None:
            total = total + bias
        if self.hist.shape[0] > 0:
            self.hist = np.concatenate([self.hist[1:], bx[None, :]], axis=0)
        return c * total


class KeyValueList:
    """Keys (normalised and rotated) and values of one attention layer, one entry a token."""

    def __init__(self):
        self.keys, self.values = [], []


def _attend(q_heads, kv: KeyValueList, n_kv_heads):
    """src/backend/cpu/scalar/core.c:415-433 and :647: head h reads kv head h // (H / G); the
    scores are divided by sqrt(d) (src/recipe/builders.c:244-248) and go through the softmax of
    src/backend/cpu/scalar/quants.c:1533-1546."""
    H, d = q_heads.shape
    rep = H // n_kv_heads
    out = np.zeros((H, d))
    for h in range(H):
        g = h // rep
        scores = [float(np.dot(k[g], q_heads[h])) / math.sqrt(d) for k in kv.keys]
        top = max(scores)
        weights = [math.exp(s - top) for s in scores]
        norm = sum(weights)
        for wgt, v in zip(weights, kv.values):
            out[h] += (wgt / norm) * v[g]
    return out


def forward_by_steps(cfg: dict, w: dict, tokens):
    """Logits [T, V] of a sequence, computed one token after the other (src/models/lfm.c:7-62;
    order of a step as src/recipe/exec.c:704-758)."""
    D = int(cfg["hidden_size"])
    H = int(cfg["num_attention_heads"])
    G = int(cfg["num_key_value_heads"])
    d = int(cfg.get("head_dim") or D // H)
    eps, theta = float(cfg["norm_eps"]), float(cfg["rope_theta"])
    taps = int(cfg["conv_L_cache"])
    kinds = list(cfg["layer_types"])
    table = w["model.embed_tokens.weight"].astype(np.float64)
    head = table if cfg.get("tie_embedding", True) else w["lm_head.weight"].astype(np.float64)
    state = [ConvState(D, taps) if kind == "conv" else KeyValueList() for kind in kinds]
    with_bias = bool(cfg.get("conv_bias", False))
    logits = []
    for position, token in enumerate(tokens):
        x = table[int(token)].copy()
        for i, kind in enumerate(kinds):
            p = f"model.layers.{i}."
            get = lambda name: w[p + name].astype(np.float64)
            xn = _norm(x, get("operator_norm.weight"), eps)
            if kind == "conv":
                mixed = get("conv.in_proj.weight") @ xn
                if with_bias:
                    mixed = mixed + get("conv.in_proj.bias")
                b, c, xg = mixed[:D], mixed[D:2 * D], mixed[2 * D:]        # src/backend/cpu/common.c:2401-2403
                taps_w = get("conv.conv.weight").reshape(D, taps)
                y = state[i].step(b, c, xg, taps_w, get("conv.conv.bias") if with_bias else None)
                update = get("conv.out_proj.weight") @ y
                if with_bias:
                    update = update + get("conv.out_proj.bias")
            else:
                q = (get("self_attn.q_proj.weight") @ xn).reshape(H, d)
                k = (get("self_attn.k_proj.weight") @ xn).reshape(G, d)
                v = (get("self_attn.v_proj.weight") @ xn).reshape(G, d)
                qn, kn = get("self_attn.q_layernorm.weight"), get("self_attn.k_layernorm.weight")
                # norm before rotation, one weight for all heads (src/models/lfm.c:36-39)
                q = np.stack([_rotate(_norm(q[h], qn, eps), position, theta) for h in range(H)])
                k = np.stack([_rotate(_norm(k[g], kn, eps), position, theta) for g in range(G)])
                state[i].keys.append(k)
                state[i].values.append(v)
                update = get("self_attn.out_proj.weight") @ _attend(q, state[i], G).reshape(H * d)
            x = x + update
            xn = _norm(x, get("ffn_norm.weight"), eps)
            gate = get("feed_forward.w1.weight") @ xn
            up = get("feed_forward.w3.weight") @ xn
            act = np.array([g / (1.0 + math.exp(-g)) for g in gate]) * up    # src/backend/cpu/quants.h:369-371
            x = x + get("feed_forward.w2.weight") @ act
        logits.append(head @ _norm(x, w["model.embedding_norm.weight"].astype(np.float64), eps))
    return np.stack(logits)
