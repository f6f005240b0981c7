"""A plain, slow implementation of the Lomodra decoder: one function per mechanism, whole
sequences, dense matrices, float64, token-by-token recurrences.  It shares no code with the engine.

Notation: ``x`` is the residual stream ``[T, W]``; a sublayer reads ``x`` as it is and its OUTPUT is
normed before it enters the stream: ``x <- x + n1(mixer(x))``, ``x <- x + n2(ff(x))``, and then a
per-layer input that depends on the token alone, ``x <- x + n3(P (gelu(G x) * e_token))``.  Mixers:
``lightning`` (linear attention with one fixed decay a head), ``attention`` (softmax attention inside
chunks of positions, normed queries and keys, no positions in the scores, keys and values possibly
taken from an earlier layer), ``channel_delta`` (a gated delta rule with a decay per key channel).
The feed-forward is a mixture of gated experts beside one expert that every token uses.

``rounded`` stands where a 16-bit engine rounds a value it hands on (identity for 32-bit).
"""
import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def _same(t):
    return t


def rms(x, eps):
    return torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return x / rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


# ---- mixers ---------------------------------------------------------------------------------
def lightning(W: Dict[str, torch.Tensor], p: str, m: dict, h, eps: float, rounded=_same):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q, k, v = silu of their projections; all
    heads' read-outs are normed together, gated by sigmoid(W_g h) and projected."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(rounded(h @ W[p + "q"].T)).view(T, H, d)
    k = silu(rounded(h @ W[p + "k"].T)).view(T, H, d)
    v = silu(rounded(h @ W[p + "v"].T)).view(T, H, dv)
    o = fixed_decay_steps(q, k, v, torch.tensor([float(a) for a in m["decay"]], dtype=F))
    o = rms_norm(o.reshape(T, H * dv), W[p + "norm"], eps)
    o = rounded(o * torch.sigmoid(rounded(h @ W[p + "g"].T)))
    return rounded(o @ W[p + "o"].T)


def fixed_decay_steps(q, k, v, decay):
    """q, k [T, H, d], v [T, H, dv], decay [H]: S_t = decay_h S_(t-1) + k_t v_t^T from S = 0; returns o_t = S_t^T q_t."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F)
    o = torch.zeros(T, H, v.shape[2], dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o


def chunk_mask(T: int, size: Optional[int]):
    """[T, T] True where query i sees key j: j <= i and, with chunks, both in the same chunk of
    ``size`` positions counted from 0."""
    i = torch.arange(T)
    see = i[None, :] <= i[:, None]
    if size:
        see = see & ((i[None, :] // size) == (i[:, None] // size))
    return see


def attention_keys_values(W, p: str, m: dict, h, eps: float, rounded=_same):
    """What an attention layer keeps per token: its normed keys [T, G, d] and its values [T, G, dv]."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rounded(h @ W[p + "k"].T).view(T, G, d)
    k = rounded(rms_norm(k, W[p + "k.norm"], eps))
    v = rounded(h @ W[p + "v"].T).view(T, G, dv)
    return k, v


def attention(W, p: str, m: dict, h, eps: float, kv, rounded=_same):
    """Grouped-query softmax attention inside chunks; ``kv`` = (keys, values) of this layer or of the
    layer it takes them from."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rounded(h @ W[p + "q"].T).view(T, H, d)
    q = rounded(rms_norm(q, W[p + "q.norm"], eps))
    k, v = kv
    out = softmax_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size"))
    return rounded(rounded(out.reshape(T, H * dv)) @ W[p + "o"].T)


def softmax_attention(q, k, v, scale: float, size: Optional[int]):
    """q [T, H, d], k [T, G, d], v [T, G, dv]: softmax((q . k) scale) over the keys ``chunk_mask`` shows, times v."""
    T, H = q.shape[:2]
    G = k.shape[1]
    see = chunk_mask(T, size)
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for hq in range(H):
        g = hq // (H // G)
        s = ((q[:, hq] @ k[:, g].T) * scale).masked_fill(~see, float("-inf"))
        out[:, hq] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def causal_conv(x, w):
    """x [T, C], w [C, taps] (last column the current token's); zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], 0)
    out = torch.zeros_like(x)
    for j in range(taps):
        out = out + pad[j:j + T] * w[:, j]
    return out


def delta_rule_steps(q, k, v, beta, g):
    """q, k [T, G, d] (already unit vectors), v [T, H, dv], beta [T, H], g [T, H, d]; from S = 0, per head and
    token in this order: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, G, d = q.shape
    H, dv = v.shape[1], v.shape[2]
    S = torch.zeros(H, d, dv, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        for hh in range(H):
            kk, qq = k[t, hh // (H // G)], q[t, hh // (H // G)]
            S[hh] = g[t, hh][:, None] * S[hh]
            u = beta[t, hh] * (v[t, hh] - S[hh].T @ kk)
            S[hh] = S[hh] + kk[:, None] * u[None, :]
            o[t, hh] = S[hh].T @ qq
    return o


def channel_delta(W, p: str, m: dict, h, eps: float, rounded=_same):
    """Gated delta rule whose decay has one value per head and key channel."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(rounded(h @ W[p + "q"].T), W[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(rounded(h @ W[p + "k"].T), W[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(rounded(h @ W[p + "v"].T), W[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(rounded(h @ W[p + "b"].T))                                    # [T, H]
    z = rounded(h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]                   # [T, H d]
    g = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * softplus(z).view(T, H, d))
    o = delta_rule_steps(q, k, v, beta, g)
    o = o / rms(o, eps) * W[p + "norm"]
    gate = torch.sigmoid(rounded(rounded(h @ W[p + "g1"].T) @ W[p + "g2"].T)).view(T, H, dv)
    return rounded(rounded((o * gate).reshape(T, H * dv)) @ W[p + "o"].T)


# ---- feed-forward ---------------------------------------------------------------------------
def gated_expert(W, p: str, h, rounded=_same):
    return rounded(rounded(silu(rounded(h @ W[p + "gate"].T)) * rounded(h @ W[p + "up"].T)) @ W[p + "down"].T)


def router_logits(W, p: str, h):
    return h @ W[p + "router"].T + W[p + "router.b"]


def mixture(W, p: str, mlp: dict, h, rounded=_same, choices=None, margin_out=None):
    """The ``top`` experts with the largest logits, weighted by the softmax over those logits alone,
    plus the expert every token uses.  ``choices`` [T, top] overrides the router's own choice;
    ``margin_out`` (a list) receives (own choice, logit gap between the last chosen and the first
    left-out expert)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = router_logits(W, p, h)
    own = torch.topk(z, top, dim=-1).indices
    if margin_out is not None:
        ordered = torch.sort(z, dim=-1, descending=True).values
        gap = ordered[:, top - 1] - ordered[:, top] if top < E else torch.full((h.shape[0],), float("inf"), dtype=F)
        margin_out.append((own, gap))
    idx = own if choices is None else choices.long()
    wgt = torch.softmax(torch.gather(z, 1, idx), dim=-1)
    out = torch.zeros_like(h)
    for e in range(E):
        hit = (idx == e)
        rows = hit.any(-1).nonzero().flatten()
        if rows.numel():
            y = gated_expert(W, f"{p}e{e}.", h[rows], rounded)
            out[rows] += (wgt[rows] * hit[rows]).sum(-1, keepdim=True) * y
    if mlp.get("shared") is not None:
        out = out + gated_expert(W, p + "shared.", h, rounded)
    return out


# ---- per-layer token input --------------------------------------------------------------------
def token_side(W, layer: int, dim: int, x, h, tokens, eps: float, rounded=_same):
    """x + n(P (gelu(G h) * e)) with e the layer's part of the token's row of the side table."""
    p = f"l{layer}.side."
    e = W["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = rounded(gelu_tanh(rounded(h @ W[p + "gate"].T)) * e)
    y = rounded(g @ W[p + "proj"].T)
    return x + y / rms(y, eps) * W[p + "norm"]


# ---- the model ----------------------------------------------------------------------------------
def to_f64(state: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.to(F) for k, v in state.items()}


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], rounded=_same, forced=None,
            layer_outputs: Optional[list] = None, margins: Optional[dict] = None):
    """Logits [T, vocab] of one whole sequence.  ``W`` holds float64 tensors by name.  ``forced`` maps
    a layer index to the experts [T, top] its tokens are sent to (else the router decides);
    ``margins`` receives per layer (the router's own choice, its margin)."""
    choices = forced
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][tokens].clone()
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        h = rounded(x)
        if layer["type"] == "lightning":
            y = lightning(W, p, m, h, eps, rounded)
        elif layer["type"] == "channel_delta":
            y = channel_delta(W, p, m, h, eps, rounded)
        else:
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(W, p, m, h, eps, rounded)
            y = attention(W, p, m, h, eps, kept[i if m.get("kv_from") is None else m["kv_from"]], rounded)
        x = x + rms_norm(y, W[f"l{i}.norm1"], eps)
        if layer.get("mlp") is not None:
            got = [] if margins is not None else None
            y = mixture(W, f"l{i}.mlp.", layer["mlp"], rounded(x), rounded, None if choices is None else choices.get(i), got)
            if got:
                margins[i] = got[0]
            x = x + rms_norm(rounded(y), W[f"l{i}.norm2"], eps)
        if cfg.get("token_side") is not None:
            x = token_side(W, i, int(cfg["token_side"]["dim"]), x, rounded(x), tokens, eps, rounded)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    logits = rms_norm(x, W["final.norm"], eps) @ W["embed"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap > 0 else logits
