"""Whole-sequence LFM2 forward pass in float64 numpy: one function per part.

All citations are paths below the reference checkout of System64fumo/kappai.
Everything works on a whole sequence at once and nothing is cached: position ``t`` of a
sequence is simply row ``t``.
"""
from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np


# --------------------------------------------------------------------------------------
# model folder reading (the plain side has its own reader on purpose)
# --------------------------------------------------------------------------------------
def read_safetensors(path) -> dict:
    """Container rules as src/safetensors.c:9-66: u64 little-endian header length, a JSON
    header ``{name: {dtype, shape, data_offsets}}`` (``__metadata__`` skipped), then raw
    little-endian data.  bf16 is widened to float64 exactly (src/weights.c:115-133)."""
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        buf = raw[base + lo:base + hi]
        dt = info["dtype"]
        if dt == "BF16":
            u16 = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            arr = u16.view(np.float32).astype(np.float64)
        elif dt == "F32":
            arr = np.frombuffer(buf, dtype="<f4").astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(buf, dtype="<f2").astype(np.float64)
        elif dt == "I32":
            arr = np.frombuffer(buf, dtype="<i4").copy()
        else:
            raise ValueError(f"plain reader: dtype {dt} of {name}")
        out[name] = arr.reshape(info["shape"])
    return out


def read_model_dir(model_dir):
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    return cfg, read_safetensors(model_dir / "model.safetensors")


# --------------------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------------------
def feed_forward_width(cfg: dict) -> int:
    """Width of the SwiGLU hidden layer.  kappai reads it ready-made from
    ``feed_forward_length`` (src/model.c:2329-2350); a config.json gives ``block_ff_dim``
    (or, in its place, ``intermediate_size``) = I and, unless ``block_auto_adjust_ff_dim`` is
    false, asks for F = floor(2I/3); a ``block_ffn_dim_multiplier`` (1.0 when the key is
    absent) multiplies F, which is then rounded up to a multiple of ``block_multiple_of``; a
    multiplier of null does neither."""
    inter = cfg.get("block_ff_dim")
    inter = int(cfg["intermediate_size"] if inter is None else inter)
    if not cfg.get("block_auto_adjust_ff_dim", True):
        return inter
    f = (2 * inter) // 3
    mult = cfg.get("block_ffn_dim_multiplier", 1.0)
    if mult is None:
        return f
    f = int(mult * f)
    m = int(cfg.get("block_multiple_of", 256))
    return -(-f // m) * m


def rmsnorm(x, w, eps):
    """y = x * 1/sqrt(mean(x^2) + eps) * w, eps inside the root, weight after
    (src/backend/cpu/scalar/quants.c:1507-1512)."""
    ss = np.mean(x * x, axis=-1, keepdims=True)
    return x * (1.0 / np.sqrt(ss + eps)) * w


def per_head_rmsnorm(x, w, eps):
    """x: [T, heads, d]; every head is normalised over its d values with one shared
    weight [d] (src/backend/cpu/scalar/quants.c:1521-1531)."""
    return rmsnorm(x, w, eps)


def rope_angles(positions, head_dim, theta):
    """angle[p, j] = p * theta^(-2j/d) for j < d/2 (src/compute.c:22-56: column j has
    frequency theta_scale^j with theta_scale = theta^(-2/d))."""
    half = head_dim // 2
    freq = np.power(float(theta), -2.0 * np.arange(half, dtype=np.float64) / head_dim)
    return np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]


def rope_neox(x, positions, theta):
    """Rotate-half pairing (j, j + d/2) over the full head
    (src/backend/cpu/quants.h:395-409):
    v_j' = v_j c - v_{j+d/2} s ; v_{j+d/2}' = v_j s + v_{j+d/2} c.   x: [T, heads, d]."""
    d = x.shape[-1]
    half = d // 2
    ang = rope_angles(positions, d, theta)
    c = np.cos(ang)[:, None, :]
    s = np.sin(ang)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate([lo * c - hi * s, lo * s + hi * c], axis=-1)


def softmax_rows(scores):
    """max-subtracted softmax (src/backend/cpu/scalar/quants.c:1533-1546)."""
    m = np.max(scores, axis=-1, keepdims=True)
    e = np.exp(scores - m)
    return e / np.sum(e, axis=-1, keepdims=True)


def causal_attention(q, k, v, window=None, rows=None):
    """q: [T, H, d], k/v: [T, G, d].  Row p sees keys 0..p; head h reads kv head
    h // (H/G) (src/backend/cpu/scalar/core.c:647); scores scaled by 1/sqrt(d)
    (src/recipe/builders.c:244-248); softmax then sum of values
    (src/backend/cpu/scalar/core.c:415-433).  With a window W a row sees only its last W
    keys, itself included (src/backend/cpu/scalar/core.c:636-640).  ``rows``: only these rows
    are worked out (the others stay zero), for sequences too long to afford them all."""
    T, H, d = q.shape
    G = k.shape[1]
    rep = H // G
    scale = 1.0 / math.sqrt(d)
    out = np.zeros((T, H, d), dtype=np.float64)
    which = range(T) if rows is None else sorted(int(r) for r in rows)
    for g in range(G):
        kg, vg = np.ascontiguousarray(k[:, g, :]), np.ascontiguousarray(v[:, g, :])
        for h in range(g * rep, (g + 1) * rep):
            for p in which:
                lo = 0
                if window is not None and window > 0 and p + 1 > window:
                    lo = p + 1 - window
                sc = (kg[lo:p + 1] @ q[p, h, :]) * scale
                a = softmax_rows(sc[None, :])[0]
                out[p, h, :] = a @ vg[lo:p + 1]
    return out


def gqa_attention_mixer(xb, lw, cfg, positions, rnd=lambda a: a, window=None, rows=None):
    """The attention layer's mixer in the reference's order (src/models/lfm.c:32-51):
    q,k,v projections; per-head RMSNorm of q and k with the layers' eps; NEOX RoPE on q
    and k; attention over the stored keys; output projection.  ``rnd`` marks the places
    where a reduced-precision engine rounds (identity in the exact run)."""
    T = xb.shape[0]
    H = int(cfg["num_attention_heads"])
    G = int(cfg["num_key_value_heads"])
    d = int(cfg.get("head_dim") or cfg["hidden_size"] // H)
    eps = float(cfg["norm_eps"])
    theta = float(cfg["rope_theta"])
    q = rnd(xb @ lw["q_proj"].T).reshape(T, H, d)
    k = rnd(xb @ lw["k_proj"].T).reshape(T, G, d)
    v = rnd(xb @ lw["v_proj"].T).reshape(T, G, d)
    q = per_head_rmsnorm(q, lw["q_layernorm"], eps)
    k = per_head_rmsnorm(k, lw["k_layernorm"], eps)
    q = rnd(rope_neox(q, positions, theta))
    k = rnd(rope_neox(k, positions, theta))
    o = rnd(causal_attention(q, k, v, window=window, rows=rows)).reshape(T, H * d)
    return rnd(o @ lw["out_proj"].T)


def causal_short_conv(bx, w, bias=None):
    """Depthwise causal FIR over a whole sequence (src/backend/cpu/common.c:2393-2431):
    s_t[c] = sum_k w[c,k] * bx_{t-(L-1)+k}[c]; w[c, L-1] meets the current token, w[c, 0]
    the oldest, and whatever lies before the sequence counts as zero
    (src/recipe/ops_hybrid.c:353-354).   bx: [T, D], w: [D, L]."""
    T, D = bx.shape
    L = w.shape[1]
    s = np.zeros((T, D), dtype=np.float64)
    for t in range(T):
        for k in range(L):
            src = t - (L - 1) + k
            if src >= 0:
                s[t] += w[:, k] * bx[src]
    if bias is not None:
        s = s + bias
    return s


def short_conv_mixer(xb, lw, cfg, rnd=lambda a: a):
    """The conv layer's mixer (src/models/lfm.c:13-19, src/backend/cpu/common.c:2401-2403):
    p = W_in xb; split in this order B, C, x; bx = B*x; s = FIR(bx); y = C*s; out = W_out y.
    The reference has no biases; with ``conv_bias`` each of the three linear maps gets one
    (in_proj, the FIR before the C gate, out_proj)."""
    D = int(cfg["hidden_size"])
    p = xb @ lw["in_proj"].T
    if lw.get("in_proj_bias") is not None:
        p = p + lw["in_proj_bias"]
    p = rnd(p)
    Bg, Cg, xg = p[:, :D], p[:, D:2 * D], p[:, 2 * D:]
    bx = Bg * xg
    s = causal_short_conv(bx, lw["conv"], lw.get("conv_bias"))
    y = rnd(Cg * s)
    out = y @ lw["out_proj"].T
    if lw.get("out_proj_bias") is not None:
        out = out + lw["out_proj_bias"]
    return rnd(out)


def silu(z):
    """z / (1 + exp(-z)) (src/backend/cpu/quants.h:369-371)."""
    return z / (1.0 + np.exp(-z))


def swiglu_feed_forward(xb, lw, rnd=lambda a: a):
    """g = W1 xb, u = W3 xb, a = silu(g)*u, y = W2 a
    (src/recipe/builders.c:344-370,383-386)."""
    g = rnd(xb @ lw["w1"].T)
    u = rnd(xb @ lw["w3"].T)
    a = rnd(silu(g) * u)
    return rnd(a @ lw["w2"].T)


# --------------------------------------------------------------------------------------
# weights by name
# --------------------------------------------------------------------------------------
def layer_kinds(cfg):
    """layer i is a conv layer or an attention layer (src/model.c:2384-2389 marks conv
    layers by a zero kv-head count; config.json names them in ``layer_types``)."""
    kinds = []
    for t in cfg["layer_types"]:
        if t == "conv":
            kinds.append("conv")
        elif t in ("full_attention", "attention"):
            kinds.append("attention")
        else:
            raise ValueError(f"layer type {t!r}")
    assert len(kinds) == int(cfg["num_hidden_layers"])
    return kinds


def layer_weights(w, i, kind, cfg):
    p = f"model.layers.{i}."
    lw = {
        "operator_norm": w[p + "operator_norm.weight"],
        "ffn_norm": w[p + "ffn_norm.weight"],
        "w1": w[p + "feed_forward.w1.weight"],
        "w3": w[p + "feed_forward.w3.weight"],
        "w2": w[p + "feed_forward.w2.weight"],
    }
    if kind == "conv":
        lw["in_proj"] = w[p + "conv.in_proj.weight"]
        cw = w[p + "conv.conv.weight"]
        lw["conv"] = cw.reshape(cw.shape[0], cw.shape[-1])
        lw["out_proj"] = w[p + "conv.out_proj.weight"]
        if cfg.get("conv_bias", False):
            lw["in_proj_bias"] = w[p + "conv.in_proj.bias"]
            lw["conv_bias"] = w[p + "conv.conv.bias"]
            lw["out_proj_bias"] = w[p + "conv.out_proj.bias"]
    else:
        for n in ("q_proj", "k_proj", "v_proj", "out_proj"):
            lw[n] = w[p + f"self_attn.{n}.weight"]
        lw["q_layernorm"] = w[p + "self_attn.q_layernorm.weight"]
        lw["k_layernorm"] = w[p + "self_attn.k_layernorm.weight"]
    return lw


# --------------------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------------------
def rows_needed(kinds, taps: int, rows):
    """For each layer the rows of its output that the logits at ``rows`` depend on without
    going through a later attention layer's keys and values: a conv layer needs the ``taps - 1``
    rows before each row it is asked for, an attention layer the keys and values of all rows,
    hence everything before it whole (None)."""
    need, cur = [None] * len(kinds), set(int(r) for r in rows)
    for i in reversed(range(len(kinds))):
        need[i] = cur
        if cur is None or kinds[i] == "attention":
            cur = None
        else:
            cur = {r - j for r in cur for j in range(taps) if r - j >= 0}
    return need


def forward(cfg: dict, w: dict, tokens, rnd=lambda a: a, return_hidden=False, rows=None):
    """Logits [T, V] of one whole sequence.

    ``rows``: only the logits at these rows are wanted (the others come back as NaN): an
    attention layer then works out only the rows that these depend on (``rows_needed``), which
    makes a sequence of tens of thousands of tokens affordable when only the last attention
    layer has many keys to walk for few rows.  Everything that costs time in proportion to the
    length (norms, projections, the FIR, the feed-forward) still runs over all rows.

    Order as src/recipe/exec.c:704-758: embedding rows without scale
    (src/recipe/scratch.c:195-235); per layer (src/models/lfm.c:7-62 with the tail of
    src/recipe/builders.c:378-388): x += mixer(norm(x)); x += ffn(norm(x)); then the final
    norm (``embedding_norm``, src/model.c:2552-2554) and the output head, which is the
    embedding table when tied (src/model.c:2562-2571).  ``rnd`` rounds the values that a
    reduced-precision engine stores between kernels; the residual sum stays exact."""
    tokens = np.asarray(tokens, dtype=np.int64)
    T = tokens.shape[0]
    eps = float(cfg["norm_eps"])
    positions = np.arange(T)
    E = w["model.embed_tokens.weight"]
    x = E[tokens].astype(np.float64)
    kinds = layer_kinds(cfg)
    need = [None] * len(kinds) if rows is None else rows_needed(kinds, int(cfg["conv_L_cache"]),
                                                                rows)
    for i, kind in enumerate(kinds):
        lw = layer_weights(w, i, kind, cfg)
        xb = rnd(rmsnorm(x, lw["operator_norm"], eps))
        if kind == "conv":
            x = x + short_conv_mixer(xb, lw, cfg, rnd)
        else:
            x = x + gqa_attention_mixer(xb, lw, cfg, positions, rnd, rows=need[i])
        xb = rnd(rmsnorm(x, lw["ffn_norm"], eps))
        x = x + swiglu_feed_forward(xb, lw, rnd)
    if return_hidden:
        return x
    xb = rnd(rmsnorm(x, w["model.embedding_norm.weight"], eps))
    head = E if cfg.get("tie_embedding", True) else w["lm_head.weight"]
    if rows is None:
        return xb @ head.T
    logits = np.full((T, head.shape[0]), np.nan)
    wanted = sorted(int(r) for r in rows)
    logits[wanted] = xb[wanted] @ head.T
    return logits


def round_bf16(a):
    """Round float64 values to the nearest bfloat16 (ties to even), returned as float64."""
    f = np.asarray(a, dtype=np.float32)
    u = f.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32).astype(np.float64)
