"""A plain, slow Bonusun: one function per mechanism, whole sequences, float64, token-by-token
recurrences, dense masked attention.  It shares no code with the engine; the tests compare the
engine against it.

The design: a decoder whose layers are pre-norm (layer norms with weight and bias) around a mixer
and a feed-forward, whose branches enter the stream times a constant or - with ``streams`` -
through hyper-connections over several copies of the stream; mixers: softmax attention with
normed queries and keys, a partial rotation, a window and a sink (``attention``), such an
attention beside a matrix memory with exponential gates (``parallel``), a real-gated linear
recurrent unit behind a short convolution (``rglru``); feed-forwards: dense or a mixture of
clamped gated experts with a sigmoid router that chooses inside the best groups.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

F = torch.float64
# what a 16-bit engine rounds on its way (projections' results, what the output projections read, the
# experts' middles): the identity, except while ``forward(rounded=...)`` estimates what rounding does
_r = lambda t: t  # noqa: E731


def to_f64(state: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in state.items()}


def load_model_dir(path: str):
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    W = {}
    with safe_open(os.path.join(path, "model.safetensors"), "pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            W[name] = t.to(F) if t.is_floating_point() else t
    return cfg, W


# ---------------------------------------------------------------- small functions
def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def layer_norm(x, w, b, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate(x, positions, dims, base, factor=1.0):
    """x [T, heads, dim]: the first ``dims`` elements of each head, element i paired with i + dims / 2."""
    if not dims:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F) / factor
    a = positions.to(F)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- attention
def attention(h, Wt, p, m, eps, window: Optional[int]):
    """Softmax attention with normed q and k, rotation of the heads' first elements, an optional
    window and a sink per head.  ``h`` [T, width], ``p`` the tensors' prefix, ``m`` the sizes."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = _r(h @ Wt[p + "q"].T).view(T, H, d)
    k = _r(h @ Wt[p + "k"].T).view(T, G, d)
    v = _r(h @ Wt[p + "v"].T).view(T, G, dv)
    q = rms(q, eps) * Wt[p + "q.norm"]
    k = rms(k, eps) * Wt[p + "k.norm"]
    rot = m.get("rot")
    if rot:
        pos = torch.arange(T)
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotate(q, pos, int(rot["dims"]), float(rot["base"]), factor)
        k = rotate(k, pos, int(rot["dims"]), float(rot["base"]), factor)
    q, k = _r(q), _r(k)
    out = torch.zeros(T, H, dv, dtype=F)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if window:
        seen = seen & (i - j < window)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~seen, -math.inf)
        sink = Wt[p + "sink"][head]
        top = torch.maximum(s.max(-1, keepdim=True).values, sink)
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True) + torch.exp(sink - top)
        out[:, head] = (e / den) @ v[:, g]
    return _r(out.reshape(T, H * dv)) @ Wt[p + "o"].T


# ---------------------------------------------------------------- matrix memory
def matrix_memory(h, Wt, p, m, eps):
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = _r(h @ Wt[p + "q"].T).view(T, H, d) * d ** -0.5
    k = _r(h @ Wt[p + "k"].T).view(T, H, d)
    v = _r(h @ Wt[p + "v"].T).view(T, H, dv)
    gi = cap * torch.tanh((h @ Wt[p + "i"].T + Wt[p + "i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ Wt[p + "f"].T + Wt[p + "f.b"]) / cap))
    S = torch.zeros(H, d, dv, dtype=F)
    n = torch.zeros(H, d, dtype=F)
    mx = torch.zeros(H, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        new = torch.maximum(gf[t] + mx, gi[t])
        keep, take = torch.exp(gf[t] + mx - new), torch.exp(gi[t] - new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = num / den[:, None]
    o = rms(o, eps).reshape(T, H * dv) * Wt[p + "norm"]
    o = o * torch.sigmoid(_r(h @ Wt[p + "g"].T))
    return _r(o) @ Wt[p + "o"].T


# ---------------------------------------------------------------- real-gated linear recurrent unit
def rglru(h, Wt, p, m):
    T = h.shape[0]
    width, blocks, taps = m["width"], m["blocks"], m["conv"]
    y = gelu_tanh(_r(h @ Wt[p + "y"].T) + Wt[p + "y.b"])
    x = _r(h @ Wt[p + "x"].T) + Wt[p + "x.b"]
    conv = Wt[p + "conv"]                                   # [channels, taps], the last column is the current token's
    padded = torch.cat([torch.zeros(taps - 1, width, dtype=F), x], dim=0)
    u = torch.zeros(T, width, dtype=F)
    for j in range(taps):
        u = u + padded[j:j + T] * conv[:, j]
    u = u + Wt[p + "conv.b"]
    bs = width // blocks
    ub = u.view(T, blocks, bs)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, Wt[p + "ra"]) + Wt[p + "ra.b"]).reshape(T, width)
    g = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, Wt[p + "ri"]) + Wt[p + "ri.b"]).reshape(T, width)
    log_a = -8.0 * r * torch.nn.functional.softplus(Wt[p + "lam"])
    a = torch.exp(log_a)
    S = torch.zeros(width, dtype=F)
    out = torch.zeros(T, width, dtype=F)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * g[t] * u[t]
        out[t] = S
    return _r(out * y) @ Wt[p + "o"].T


# ---------------------------------------------------------------- feed-forwards
def clamped_expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return _r(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h, Wt, p, mlp, forced: Optional[torch.Tensor] = None, margins: Optional[list] = None):
    """(chosen experts [T, top], weights [T, top], choice scores [T, experts] with the left-out groups
    at -inf).  ``forced``: experts to take instead of the router's own choice (the weights follow)."""
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h @ Wt[p + "router"].T)
    choice = s + Wt[p + "correction"]
    groups = r.get("groups")
    if groups:
        cnt, keep = int(groups["count"]), int(groups["keep"])
        per = E // cnt
        gs = choice.view(-1, cnt, per).topk(min(2, per), dim=-1).values.sum(-1)
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(h.shape[0], cnt, dtype=torch.bool)
        allowed.scatter_(1, best, True)
        choice = choice.masked_fill(~allowed[:, :, None].expand(-1, -1, per).reshape(-1, E), -math.inf)
    best = choice.topk(min(top + 1, E), dim=-1)
    own = best.indices[:, :top]
    if margins is not None:
        # how clear the choice was: the gap between the last expert taken and the first one left out, and -
        # with groups - between the last group kept and the first one dropped
        gap = (best.values[:, top - 1] - best.values[:, top]) if E > top else torch.full((h.shape[0],), math.inf, dtype=F)
        gap = torch.where(torch.isfinite(gap), gap, torch.full_like(gap, math.inf))
        if groups and int(groups["keep"]) < int(groups["count"]):
            g2 = gs.topk(int(groups["keep"]) + 1, dim=-1).values
            gap = torch.minimum(gap, g2[:, -2] - g2[:, -1])
        margins.append((own, gap))
    idx = own if forced is None else forced.long()
    w = s.gather(1, idx)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))
    return idx, w, choice


def mixture(h, Wt, p, mlp, forced: Optional[torch.Tensor] = None, margins: Optional[list] = None):
    idx, w, _ = route(h, Wt, p, mlp, forced, margins)
    limit = float(mlp["expert"]["limit"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(idx.shape[1]):
            e = int(idx[t, c])
            out[t] += w[t, c] * clamped_expert(h[t:t + 1], Wt[f"{p}e{e}.gate"], Wt[f"{p}e{e}.up"],
                                               Wt[f"{p}e{e}.down"], limit)[0]
    shared = mlp.get("shared")
    if shared:
        y = _r(clamped_expert(h, Wt[p + "shared.gate"], Wt[p + "shared.up"], Wt[p + "shared.down"], float(shared["limit"])))
        out = out + y * torch.sigmoid(h @ Wt[p + "shared.sg"].T)
    return out


def dense(h, Wt, p):
    return _r(gelu_tanh(_r(h @ Wt[p + "up"].T))) @ Wt[p + "down"].T


# ---------------------------------------------------------------- the model
def run_order(cfg) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def mixer(cfg, Wt, i, h):
    layer = cfg["layers"][i]
    p, m, eps = f"l{i}.mix.", layer["mixer"], float(cfg["norm"]["eps"])
    if layer["type"] == "attention":
        return attention(h, Wt, p, m, eps, int((m.get("mask") or {}).get("size", 0)))
    if layer["type"] == "rglru":
        return rglru(h, Wt, p, m)
    left = attention(h, Wt, p + "left.", m["left"], eps, int((m["left"].get("mask") or {}).get("size", 0)))
    right = matrix_memory(h, Wt, p + "right.", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def feed_forward(cfg, Wt, i, h, forced=None, margins=None):
    mlp = cfg["layers"][i]["mlp"]
    if mlp["kind"] == "dense":
        return dense(h, Wt, f"l{i}.mlp.")
    return mixture(h, Wt, f"l{i}.mlp.", mlp, forced, margins)


def forward(cfg, Wt: Dict[str, torch.Tensor], tokens, forced: Optional[dict] = None, layers_out: Optional[list] = None,
            margins: Optional[dict] = None, rounded=None):
    """Logits [T, vocab] of a whole sequence.  ``forced``: {run index: experts [T, top]} to take in
    place of the routers' own choices; ``layers_out`` receives the stream after every layer run;
    ``margins`` receives {run index: (the router's own choice, how clear it was)}; ``rounded`` is
    applied to every branch's input and output (what a 16-bit engine rounds there)."""
    global _r
    rounded = rounded or (lambda t: t)
    _r = rounded
    try:
        return _forward(cfg, Wt, tokens, forced, layers_out, margins, rounded)
    finally:
        _r = lambda t: t  # noqa: E731


def _forward(cfg, Wt, tokens, forced, layers_out, margins, rounded):
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    S = cfg.get("streams")
    x = Wt["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = [x.clone() for _ in range(int(S))] if S else None

    def sublayer(q: int, i: int, fn):
        nonlocal x, xs
        p = f"l{i}."
        w, b = Wt[f"{p}norm{q}"], Wt[f"{p}norm{q}.b"]
        if xs is None:
            x = x + mult * rounded(fn(rounded(layer_norm(x, w, b, eps))))
            return
        u = sum(Wt[f"{p}hc{q}.in"][s] * xs[s] for s in range(len(xs)))
        y = rounded(fn(rounded(layer_norm(u, w, b, eps))))
        mix, out = Wt[f"{p}hc{q}.mix"], Wt[f"{p}hc{q}.out"]
        xs = [sum(mix[s, t] * xs[s] for s in range(len(xs))) + mult * out[t] * y for t in range(len(xs))]

    for run, i in enumerate(run_order(cfg)):
        sublayer(1, i, lambda h: mixer(cfg, Wt, i, h))
        if cfg["layers"][i].get("mlp") is not None:
            seen = [] if margins is not None else None
            sublayer(2, i, lambda h: feed_forward(cfg, Wt, i, h, None if forced is None else forced.get(run), seen))
            if seen:
                margins[run] = seen[0]
        if layers_out is not None:
            layers_out.append(x.clone() if xs is None else sum(xs))
    if xs is not None:
        x = sum(xs)
    return rounded(layer_norm(x, Wt["final.norm"], Wt["final.norm.b"], eps)) @ Wt["head"].T


def generate(cfg, Wt, prompt, new_tokens: int) -> List[int]:
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(forward(cfg, Wt, toks)[-1].argmax()))
    return toks[len(prompt):]
