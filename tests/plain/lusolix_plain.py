"""A plain, slow implementation of the Lusolix decoder on the CPU, one function per mechanism.

It shares no code with the engine: it reads a config dictionary and a dictionary of tensors and
computes a whole sequence at once with ordinary tensor expressions. ``dtype`` says what the engine's
storage type is; the places where the engine rounds to it are the places where ``rnd`` is applied
here (matrices' results, the inputs of products), everything else is 32-bit.

Notation: x is the residual stream [T, W]; n = layer_norm(x); g = sigmoid(R n + r) the residual gate;
u = n + conv(n) the mixer's input; H heads, per head Dn channels without and Dr with rotation, values of
Dv, latent of Lk channels, query latent of Lq.
"""
from __future__ import annotations

import math

import torch


def rnd(t: torch.Tensor, dtype) -> torch.Tensor:
    return t.to(dtype).float()


def linear(x, w, b=None, dtype=torch.float32):
    y = rnd(x, dtype) @ w.float().T
    if b is not None:
        y = y + b.float()
    return y


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w.float() + b.float()


def rms_norm(x, w, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w.float()


def short_conv(h, w, before=None):
    """h [T, W], w [W, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j); ``before``: the taps - 1 rows that
    came before h (zeros at a sequence's start). Returns (h + conv(h), the last taps - 1 rows seen)."""
    taps = w.shape[1]
    T, W = h.shape
    if before is None:
        before = torch.zeros((taps - 1, W))
    ext = torch.cat([before, h], 0)
    out = torch.zeros_like(h)
    for j in range(taps):
        out = out + w[:, j].float() * ext[j:j + T]
    return h + out, ext[ext.shape[0] - (taps - 1):]


def rotate_interleaved(v, positions, base, dims):
    """v [T, ..., D]: channels (2i, 2i+1), i < dims/2, turn by positions * base^(-2i/dims); the rest stay."""
    out = v.clone()
    i = torch.arange(dims // 2, dtype=torch.float32)
    f = 1.0 / (base ** (2 * i / dims))
    a = positions.float()[:, None] * f[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [dims // 2]
    c, s = a.cos().view(shape), a.sin().view(shape)
    x, y = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = x * c - y * s
    out[..., 1:dims:2] = y * c + x * s
    return out


def latent_attention(u, positions, m, t, pre, eps, dtype, seen=None):
    """u [T, W]: the mixer's input; m: the mixer's sizes; t: tensors; pre: the mixer's prefix.
    ``seen``: (latents, rotated shared keys, their positions) of earlier tokens of the sequence.
    Returns (output [T, W], (latents, shared keys, positions) with this call's appended)."""
    H, Dn, Dr, Dv, Lk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = u.shape[0]
    cq = rms_norm(linear(u, t[pre + "dq"], None, dtype), t[pre + "dq.norm"], eps)
    q = rnd(linear(cq, t[pre + "uq"], None, dtype), dtype).view(T, H, Dn + Dr)
    low = linear(u, t[pre + "dkv"], None, dtype)
    c = rnd(rms_norm(low[:, :Lk], t[pre + "dkv.norm"], eps), dtype)
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    kr = low[:, Lk:]
    qn, qr = q[..., :Dn], q[..., Dn:]
    if dims:
        kr = rotate_interleaved(kr, positions, float(rot["base"]), dims)
        qr = rotate_interleaved(qr, positions, float(rot["base"]), dims)
    kr = rnd(kr, dtype)
    if seen is not None:
        c_all, kr_all, p_all = torch.cat([seen[0], c]), torch.cat([seen[1], kr]), torch.cat([seen[2], positions])
    else:
        c_all, kr_all, p_all = c, kr, positions
    uk = t[pre + "uk"].float().view(H, Dn, Lk)
    uv = t[pre + "uv"].float().view(H, Dv, Lk)
    kn = torch.einsum("jl,hdl->jhd", c_all, uk)
    val = torch.einsum("jl,hdl->jhd", c_all, uv)
    score = (torch.einsum("thd,jhd->htj", qn, kn) + torch.einsum("thd,jd->htj", qr, kr_all)) * float(m["scale"])
    dist = positions[:, None] - p_all[None, :]
    size = (m.get("mask") or {}).get("size")
    ok = dist >= 0
    if size:
        ok = ok & (dist < int(size))
    score = score.masked_fill(~ok[None], float("-inf"))
    wgt = torch.softmax(score, -1)
    o = torch.einsum("htj,jhd->thd", wgt, val)
    gate = torch.sigmoid(linear(u, t[pre + "g"], None, dtype))              # [T, H]
    o = rnd(o * gate[:, :, None], dtype).reshape(T, H * Dv)
    return linear(o, t[pre + "o"], None, dtype), (c_all, kr_all, p_all)


def poly_norm(z, coef, eps):
    a, b, c, e = [float(v) for v in coef.float()]
    return a * rms_norm(z, None, eps) + b * rms_norm(z * z, None, eps) + c * rms_norm(z * z * z, None, eps) + e


def dense_ff(n, t, pre, eps, dtype):
    z = linear(n, t[pre + "up"], None, dtype)
    return linear(poly_norm(z, t[pre + "act"], eps), t[pre + "down"], None, dtype)


def table_experts(n, token_ids, t, pre, dtype):
    """Every token's experts come from a table row of its id; each weighs 1 / (entries in a row)."""
    table = t[pre + "table"].long()
    top = table.shape[1]
    out = torch.zeros((n.shape[0], t[pre + "e0.down"].shape[0]))
    for i in range(n.shape[0]):
        for k in range(top):
            e = int(table[int(token_ids[i]), k])
            p = f"{pre}e{e}."
            gt = linear(n[i:i + 1], t[p + "gate"], None, dtype)
            up = linear(n[i:i + 1], t[p + "up"], None, dtype)
            out[i] += linear(torch.nn.functional.silu(gt) * up, t[p + "down"], None, dtype)[0] / top
    return out


def forward(cfg: dict, t: dict, token_ids, dtype=torch.float32, start: int = 0, state: dict | None = None,
            trace: list | None = None):
    """Logits [T, vocab] of the tokens at positions start .. start + T - 1; ``state`` carries a sequence from one call
    to the next (pass the same dictionary again). ``trace`` collects the residual stream after every layer."""
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    T = ids.numel()
    pos = torch.arange(start, start + T)
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = t["embed"].float()[ids] + t["pos"].float()[pos]
    state = state if state is not None else {}
    for i, layer in enumerate(cfg["layers"]):
        L = f"l{i}."
        n = rnd(layer_norm(x, t[L + "norm1"], t[L + "norm1.b"], eps), dtype)
        g = torch.sigmoid(rnd(linear(n, t[L + "rg1"], t[L + "rg1.b"], dtype), dtype))
        u = n
        if L + "canon1" in t:
            u, state[L + "conv"] = short_conv(n, t[L + "canon1"], state.get(L + "conv"))
            u = rnd(u, dtype)
        y, state[L + "kv"] = latent_attention(u, pos, layer["mixer"], t, L + "mix.", eps, dtype, state.get(L + "kv"))
        x = x + mult * (rnd(y, dtype) * g)
        mlp = layer.get("mlp")
        if mlp is not None:
            n = rnd(layer_norm(x, t[L + "norm2"], t[L + "norm2.b"], eps), dtype)
            g = torch.sigmoid(rnd(linear(n, t[L + "rg2"], t[L + "rg2.b"], dtype), dtype))
            if mlp.get("kind", "dense") == "dense":
                y = dense_ff(n, t, L + "mlp.", eps, dtype)
            else:
                y = table_experts(n, ids, t, L + "mlp.", dtype)
            x = x + mult * (rnd(y, dtype) * g)
        if trace is not None:
            trace.append(x.clone())
    n = rnd(layer_norm(x, t["final.norm"], t["final.norm.b"], eps), dtype)
    return linear(n, t["embed"], None, dtype)
