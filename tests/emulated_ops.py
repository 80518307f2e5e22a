"""A stand-in for ``kappai_amd.kernels.ops`` made of torch CPU operations, so that the
engine's own logic (row tables, cache manager, step function, scheduler, replay) can be
tested where there is no GPU.  It belongs to the tests; the package never imports it.
Every function has the contract of the kernel it stands for, including the dtype in which
results are stored."""
from __future__ import annotations

import numpy as np
import torch

F32, BF16 = torch.float32, torch.bfloat16
ROT_NONE, ROT_HALF, ROT_INTERLEAVED = 0, 1, 2


def embed_rows(ids, table):
    return table[ids.long()].to(F32)


def add_rmsnorm(resid, delta, weight, eps, out_dtype, rows=None, write_resid=True,
                fragment=False):
    assert not fragment, "rows in fragment order are made on the GPU only"
    x = resid
    if delta is not None:
        parts = delta if delta.dim() == 3 else delta[None]
        for p in parts:                       # partial sums are added in order
            x = x + p.to(F32)
    if delta is not None and write_resid and rows is None:
        resid.copy_(x)
    if rows is not None:
        x = x[rows.long()]
    y = x * (1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)) * weight
    return y.to(out_dtype)


def sum_partial_sums(parts):
    out = parts[0].to(F32).clone()
    for p in parts[1:]:
        out += p
    return out


def add_residual(resid, delta):
    resid.add_(delta.to(F32))


def swiglu(gate_up):
    F = gate_up.shape[1] // 2
    g, u = gate_up[:, :F].to(F32), gate_up[:, F:].to(F32)
    return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)


def cast(x, dtype):
    return x.to(dtype)


def linear(x, weight, bias=None, out_dtype=None, force_kernel=0, partial_sums=False,
           split_k=None, weight_frag=None, add_into=None):
    # ``add_into`` is an offer the stand-in does not take up: the result comes back as always
    out_dtype = out_dtype or x.dtype
    y = x.to(F32) @ weight.to(F32).T
    if bias is not None:
        y = y + bias
    return y.to(out_dtype)


SWIGLU_GROUP = 16


def interleave_gate_up(gate, up):
    F, K = gate.shape
    g = gate.reshape(F // SWIGLU_GROUP, 1, SWIGLU_GROUP, K)
    u = up.reshape(F // SWIGLU_GROUP, 1, SWIGLU_GROUP, K)
    return torch.cat([g, u], dim=1).reshape(2 * F, K).contiguous()


def linear_swiglu(x, weight, force_kernel=0, weight_frag=None, out_fragment=False):
    F = weight.shape[0] // 2
    y = (x.to(F32) @ weight.to(F32).T).reshape(x.shape[0], F // SWIGLU_GROUP, 2, SWIGLU_GROUP)
    g, u = y[:, :, 0, :].reshape(-1, F), y[:, :, 1, :].reshape(-1, F)
    return (g / (1.0 + torch.exp(-g)) * u).to(x.dtype)


def shortconv(proj, taps, bias, state, row_seg, seg_start, seg_pos0, seg_slot):
    T = proj.shape[0]
    D, L = taps.shape
    H = L - 1
    p = proj.to(F32)
    B, C, X = p[:, :D], p[:, D:2 * D], p[:, 2 * D:]
    bx = B * X
    out = torch.empty((T, D), dtype=F32)
    for s in range(seg_pos0.shape[0]):
        t0, t1 = int(seg_start[s]), int(seg_start[s + 1])
        slot = int(seg_slot[s])
        hist = torch.zeros((H, D)) if int(seg_pos0[s]) == 0 else state[slot].T.clone()
        seq = torch.cat([hist, bx[t0:t1]], dim=0)            # [H + n, D]
        for r in range(t1 - t0):
            acc = torch.zeros(D) if bias is None else bias.clone()
            for k in range(L):
                acc = acc + taps[:, k] * seq[r + k]
            out[t0 + r] = C[t0 + r] * acc
        state[slot] = seq[-H:].T
    return out.to(proj.dtype)


def linear_shortconv_step(x, in_proj, in_bias, taps, conv_bias, state, seg_pos0, seg_slot,
                          weight_frag=None, out_fragment=False):
    M = x.shape[0]
    proj = linear(x, in_proj, in_bias)
    row_seg = torch.arange(M, dtype=torch.int32)
    seg_start = torch.arange(M + 1, dtype=torch.int32)
    return shortconv(proj, taps, conv_bias, state, row_seg, seg_start, seg_pos0, seg_slot)


def qk_norm_rope_store(qkv, n_heads, n_kv_heads, head_dim, q_norm_w, k_norm_w, eps, cos, sin,
                       rot_dim, rot_mode, k_pool, v_pool, row_pos, row_seg, block_tables,
                       page_size, store_kv=True):
    H, G, d = n_heads, n_kv_heads, head_dim
    T = qkv.shape[0]
    pos = row_pos.long()

    def norm_rot(x, w):                                      # x: [T, heads, d] float32
        if w is not None:
            x = x * (1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)) * w
        if rot_mode == ROT_NONE:
            return x
        half = rot_dim // 2
        c, s = cos[pos][:, None, :], sin[pos][:, None, :]
        y = x.clone()
        if rot_mode == ROT_HALF:
            a, b = x[..., :half], x[..., half:rot_dim]
            y[..., :half] = a * c - b * s
            y[..., half:rot_dim] = a * s + b * c
        else:
            a, b = x[..., 0:rot_dim:2], x[..., 1:rot_dim:2]
            y[..., 0:rot_dim:2] = a * c - b * s
            y[..., 1:rot_dim:2] = a * s + b * c
        return y

    q = norm_rot(qkv[:, :H * d].to(F32).reshape(T, H, d), q_norm_w)
    qkv[:, :H * d] = q.reshape(T, H * d).to(qkv.dtype)
    if not store_kv:
        return qkv
    k = norm_rot(qkv[:, H * d:(H + G) * d].to(F32).reshape(T, G, d), k_norm_w)
    v = qkv[:, (H + G) * d:(H + 2 * G) * d].reshape(T, G, d)
    for t in range(T):
        p = int(row_pos[t])
        page = int(block_tables[int(row_seg[t]), p // page_size])
        assert page >= 0, "a row is stored into a page that was given back"
        k_pool[page, :, p % page_size, :] = k[t].to(k_pool.dtype)
        v_pool[page, :, :, p % page_size] = v[t].to(v_pool.dtype)
    return qkv


def paged_attention(q, n_heads, n_kv_heads, head_dim, k_pool, v_pool, row_pos, row_seg,
                    block_tables, page_size, scale, window=0, **_unused):
    H, G, d = n_heads, n_kv_heads, head_dim
    T = q.shape[0]
    out = torch.empty((T, H * d), dtype=F32)
    for t in range(T):
        p = int(row_pos[t])
        lo = p + 1 - window if window and p + 1 > window else 0
        bt = block_tables[int(row_seg[t])]
        idx = torch.arange(lo, p + 1)
        pages = bt[(idx // page_size).long()].long()
        assert bool((pages >= 0).all()), "attention reads a page that was given back"
        keys = k_pool[pages, :, (idx % page_size).long(), :].to(F32)     # [n, G, d]
        vals = v_pool[pages, :, :, (idx % page_size).long()].to(F32)             # [n, G, d]
        qt = q[t, :H * d].to(F32).reshape(H, d)
        for h in range(H):
            g = h // (H // G)
            sc = (keys[:, g, :] @ qt[h]) * scale
            a = torch.softmax(sc, dim=0)
            out[t, h * d:(h + 1) * d] = a @ vals[:, g, :]
    return out.to(q.dtype)


def sample_rows(logits, temperature, uniform):
    out = torch.empty(logits.shape[0], dtype=torch.int32)
    for r in range(logits.shape[0]):
        lg = logits[r].double()
        t = float(temperature[r])
        if not t > 0:
            m = lg.max()
            out[r] = int(torch.nonzero(lg == m)[0])
            continue
        z = (logits[r] * (1.0 / t))
        e = torch.exp(z - z.max()).double()
        acc = torch.cumsum(e, 0)
        target = float(uniform[r]) * float(acc[-1])
        i = int(torch.searchsorted(acc, torch.tensor(target, dtype=torch.float64), right=True))
        out[r] = min(i, logits.shape[1] - 1)
    return out


FILTER_MAX_KEEP = 1024


def sample_filtered(logits, rows, keep, temperature, top_p, min_p, uniform, out):
    from plain import sampler as plain_sampler
    for i in range(rows.shape[0]):
        r = int(rows[i])
        k = int(keep[i])
        out[r] = plain_sampler.sample_filtered(
            logits[r].numpy(), float(temperature[i]), k if k < logits.shape[1] else 0,
            float(top_p[i]), float(min_p[i]), float(uniform[i]), cap=k)


def repeat_penalty(logits, row_start, tokens, penalty):
    for r in range(logits.shape[0]):
        pen = float(penalty[r])
        if pen == 1.0:
            continue
        for i in range(int(row_start[r]), int(row_start[r + 1])):
            tok = int(tokens[i])
            if 0 <= tok < logits.shape[1]:
                logits[r, tok] = logits[r, tok] / pen if logits[r, tok] > 0 else logits[r, tok] * pen


def history_set(history, seen, slots, starts, tokens):
    cap = history.shape[1]
    for i in range(slots.shape[0]):
        lo, hi = int(starts[i]), int(starts[i + 1])
        n = min(hi - lo, cap)
        history[int(slots[i]), :n] = tokens[lo:lo + n]
        seen[int(slots[i])] = n


def repeat_penalty_history(logits, rows, slots, penalty, last_n, history, seen):
    cap = history.shape[1]
    for i in range(rows.shape[0]):
        pen = float(penalty[i])
        if pen == 1.0:
            continue
        slot, total = int(slots[i]), int(seen[int(slots[i])])
        n = min(int(last_n[i]), total, cap)
        r = int(rows[i])
        for j in range(total - n, total):
            tok = int(history[slot, j % cap])
            if 0 <= tok < logits.shape[1]:
                logits[r, tok] = logits[r, tok] / pen if logits[r, tok] > 0 else logits[r, tok] * pen


def history_append(chosen, rows, slots, history, seen):
    cap = history.shape[1]
    for i in range(rows.shape[0]):
        slot = int(slots[i])
        history[slot, int(seen[slot]) % cap] = chosen[int(rows[i])]
        seen[slot] += 1


ALL = ["embed_rows", "add_rmsnorm", "add_residual", "sum_partial_sums", "swiglu", "cast", "linear", "linear_swiglu",
       "interleave_gate_up", "shortconv", "linear_shortconv_step",
       "qk_norm_rope_store", "paged_attention", "sample_rows", "sample_filtered",
       "repeat_penalty", "history_set", "repeat_penalty_history", "history_append"]


def install(monkeypatch):
    """Replace the kernels' Python faces by these functions for one test."""
    import sys

    from kappai_amd.kernels import ops
    me = sys.modules[__name__]
    for name in ALL:
        monkeypatch.setattr(ops, name, getattr(me, name))


def make_cpu_runner(model, cache):
    """A StepRunner whose tables stay on the host (the emulated kernels read them there)."""
    from kappai_amd.engine.step import StepRunner

    class HostTableRunner(StepRunner):
        def __init__(self, model, cache):
            super().__init__(model, cache, device="cpu")

        def _upload(self, arrays):
            return {k: torch.from_numpy(np.ascontiguousarray(v).copy()) for k, v in arrays.items()}

    return HostTableRunner(model, cache)
