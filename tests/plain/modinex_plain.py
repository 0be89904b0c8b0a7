"""The Modinex decoder written out plainly, one function per mechanism, on the CPU with torch tensor
expressions and Python loops only. It shares no code with the engine: the tests compare the two.

Notation. T tokens of one sequence at positions 0..T-1, width W. A layer is

    x <- x + N1b(mix(N1(x)));   x <- x + N2b(ff(N2(x)))       (the second line only if the layer has a feed-forward)

with N* the norm in groups. ``dt`` is the type of the matrix products' operands and results: torch.float32
computes everything in 32-bit; torch.bfloat16 rounds weights, the inputs of every product, and its result,
to bfloat16 and keeps in 32-bit what the design keeps there (norm statistics, angles, scores and weights of
the attention, the decays and the state of the recurrence, the residual stream).
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


def rnd(x: torch.Tensor, dt) -> torch.Tensor:
    """x rounded to ``dt`` and widened again."""
    return x.float() if dt == torch.float32 else x.to(dt).float()


def linear(x, w, b, dt, keep32: bool = False):
    """y = x W^T (+ b): operands rounded to dt, sums in 32-bit (64-bit here, rounded once), result rounded to dt
    unless ``keep32``."""
    y = (rnd(x, dt).double() @ rnd(w, dt).double().t())
    if b is not None:
        y = y + rnd(b, dt).double()
    y = y.float()
    return y if keep32 else rnd(y, dt)


# ------------------------------------------------------------------------------------------------ norms

def group_rms_norm(x, w, eps: float, groups: int):
    """x [.., W] cut into ``groups`` equal consecutive parts; each part divided by sqrt(mean(part^2) + eps);
    the whole times w. 32-bit."""
    shape = x.shape
    p = x.float().reshape(*shape[:-1], groups, shape[-1] // groups)
    p = p / torch.sqrt(p.pow(2).mean(-1, keepdim=True) + eps)
    return p.reshape(shape) * w.float()


def unit_rms(x, w, eps: float):
    """One vector (the last axis) divided by its root mean square, times w."""
    return group_rms_norm(x, w, eps, 1)


# ------------------------------------------------------------------------------------------------ positions

def rotate(x, pos, base: float, dims: int):
    """x [T, heads, D]; the first ``dims`` channels of each head rotate: channel i pairs with i + dims/2,
    angle pos * base^(-2i/dims). The rest passes."""
    if not dims:
        return x.float()
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = (float(base) ** (-2.0 * i / dims)).float()                      # 32-bit frequencies
    a = pos.float()[:, None] * f[None, :]                               # [T, half], 32-bit angles
    c, s = a.cos()[:, None, :], a.sin()[:, None, :]
    x = x.float()
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ------------------------------------------------------------------------------------------------ mixers

def sigmoid_attention(q, k, v, pb, scale: float, chunk: int | None, pos_q, pos_k):
    """q [Tq, H, D], k [Tk, G, D], v [Tk, G, Dv]; query head h reads kv head h // (H/G). A key at position j is
    visible from position i if j <= i and both lie in the same chunk of ``chunk`` positions counted from 0.
    Its weight is sigmoid(scale * q.k + pb[h]); the weights are not normalized. Returns [Tq, H, Dv] in 32-bit."""
    Tq, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(Tq, H, v.shape[-1])
    for h in range(H):
        g = h // rep
        s = (q[:, h].double() @ k[:, g].double().t()).float() * scale + pb[h].float()
        w = torch.sigmoid(s)
        see = pos_k[None, :] <= pos_q[:, None]
        if chunk:
            see &= (pos_k[None, :] // chunk) == (pos_q[:, None] // chunk)
        w = torch.where(see, w, torch.zeros(()))
        out[:, h] = (w.double() @ v[:, g].double()).float()
    return out


def attention_mixer(h, w, p, m, eps, dt, pos=None):
    """The attention mixer on the normed input h [T, W]; ``m`` is the layer's 'mixer' dictionary, ``p`` the
    tensor prefix ('l3.mix.')."""
    T = h.shape[0]
    pos = torch.arange(T) if pos is None else pos
    H, G, D, Dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = linear(h, w[p + "q"], None, dt).view(T, H, D)
    k = linear(h, w[p + "k"], None, dt).view(T, G, D)
    v = linear(h, w[p + "v"], None, dt).view(T, G, Dv)
    q = unit_rms(q, rnd(w[p + "q.norm"], dt), eps)
    k = unit_rms(k, rnd(w[p + "k.norm"], dt), eps)
    rot = m.get("rot") or {}
    q = rnd(rotate(q, pos, rot.get("base", 1.0), rot.get("dims", 0)), dt)
    k = rnd(rotate(k, pos, rot.get("base", 1.0), rot.get("dims", 0)), dt)
    chunk = (m.get("mask") or {}).get("size")
    o = sigmoid_attention(q, k, v, rnd(w[p + "pb"], dt), m["scale"], chunk, pos, pos)
    return linear(rnd(o, dt).reshape(T, H * Dv), w[p + "o"], None, dt)


def gla_recurrence(q, k, v, log_alpha, state=None):
    """Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t. q, k, log_alpha [T, H, D], v [T, H, Dv];
    S [H, D, Dv] in 32-bit, from zero unless given. Returns (o [T, H, Dv], S after the last token)."""
    T, H, D = k.shape
    S = torch.zeros(H, D, v.shape[-1]) if state is None else state.clone()
    o = torch.zeros(T, H, v.shape[-1])
    for t in range(T):
        S = torch.exp(log_alpha[t])[:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hd,hde->he", q[t], S)
    return o, S


def gla_mixer(h, w, p, m, eps, dt, state=None, return_state: bool = False):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (linear(h, w[p + "q"], None, dt) * D ** -0.5).view(T, H, D)
    k = linear(h, w[p + "k"], None, dt).view(T, H, D)
    v = linear(h, w[p + "v"], None, dt).view(T, H, Dv)
    z = linear(linear(h, w[p + "a1"], None, dt), w[p + "a2"], w[p + "a2.b"], dt, keep32=True).view(T, H, D)
    log_alpha = torch.nn.functional.logsigmoid(z) / float(m["tau"])       # alpha = sigmoid(z)^(1/tau)
    o, S = gla_recurrence(q, k, v, log_alpha, state)
    o = unit_rms(o, rnd(w[p + "norm"], dt), eps)                          # per head over Dv
    g = linear(h, w[p + "g"], None, dt)
    y = rnd(o.reshape(T, H * Dv) * torch.nn.functional.silu(g), dt)
    out = linear(y, w[p + "o"], None, dt)
    return (out, S) if return_state else out


# ------------------------------------------------------------------------------------------------ feed-forward

def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_ff(h, w, p, dt):
    """down(gelu_tanh(up h + b_up)) + b_down."""
    a = rnd(gelu_tanh(linear(h, w[p + "up"], w[p + "up.b"], dt)), dt)
    return linear(a, w[p + "down"], w[p + "down.b"], dt)


# ------------------------------------------------------------------------------------------------ the model

def layer(x, w, i: int, spec: dict, norm: dict, dt):
    eps, groups = norm["eps"], norm.get("groups", 1)
    p = f"l{i}."
    h = rnd(group_rms_norm(x, rnd(w[p + "norm1"], dt), eps, groups), dt)
    mix = {"attention": attention_mixer, "gla": gla_mixer}[spec["type"]](h, w, p + "mix.", spec["mixer"], eps, dt)
    x = x + group_rms_norm(mix, rnd(w[p + "norm1b"], dt), eps, groups)
    if spec.get("mlp"):
        h = rnd(group_rms_norm(x, rnd(w[p + "norm2"], dt), eps, groups), dt)
        x = x + group_rms_norm(dense_ff(h, w, p + "mlp.", dt), rnd(w[p + "norm2b"], dt), eps, groups)
    return x


def logits(w, cfg: dict, ids, dt=torch.float32, residuals: list | None = None):
    """Float32 logits [T, vocab] of one sequence from position 0. ``residuals`` collects x after every layer."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    T = ids.numel()
    x = rnd(w["embed"], dt)[ids] + rnd(w["pos"], dt)[:T]
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, w, i, spec, cfg["norm"], dt)
        if residuals is not None:
            residuals.append(x.clone())
    h = rnd(group_rms_norm(x, rnd(w["final.norm"], dt), cfg["norm"]["eps"], cfg["norm"].get("groups", 1)), dt)
    return linear(h, w["head"], None, dt, keep32=True)


def read_weights(model_dir) -> tuple[dict, dict]:
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    w = {}
    with safe_open(str(model_dir / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).float()
    return cfg, w
