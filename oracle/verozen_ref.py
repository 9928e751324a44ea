"""Plain, slow restatement of the Verozen design for checking the product path: one function per mechanism, whole
sequences at once, no cache, no state hand-over, no batching, float64 by default.  Test infrastructure only; nothing
under sglang_custom_amd/ imports it and it imports nothing from there.

Notation: x [T, D] is the residual stream of ONE sequence at positions 0..T-1; weights come in a dict under their
checkpoint names (linear weights [out, in], applied as x @ W.T).

  layer       x <- N1(c x + mixer(x));  x <- N2(c x + ff(x));  x <- x + side(x, tokens)         (c = postln_alpha)
  N           grouped RMS norm: the row is cut into `groups` equal parts, each divided by its own root mean square
  mixer       one of: gated linear attention (a decay per key channel), sigmoid attention (no softmax, values = raw keys),
              retention (a fixed decay per head)
  ff          grouped top-k mixture of erf-GELU experts with sigmoid scores and a selection-only correction
  side        a per-layer slice of a second embedding table gates a low-rank update that is RMS-normed before it is added
  output      logits = head N(x)
"""
import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------------- small pieces
def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    T, D = x.shape
    return unit_rms(x.reshape(T, groups, D // groups), eps).reshape(T, D) * w


def angles(T: int, dims: int, base: float, dtype) -> torch.Tensor:
    """[T, dims / 2]: position p times base^(-2 i / dims)."""
    i = torch.arange(dims // 2, dtype=dtype)
    return torch.arange(T, dtype=dtype)[:, None] * base ** (-2.0 * i / dims)[None, :]


def rotate_pairs(x: torch.Tensor, dims: int, base: float, neighbours: bool) -> torch.Tensor:
    """x [T, H, d]: the first `dims` features of each head are rotated by the position's angles; feature 2i goes with
    2i + 1 (neighbours) or feature i with i + dims / 2 (halves).  The rest passes."""
    if not dims:
        return x
    T = x.shape[0]
    a = angles(T, dims, base, x.dtype)[:, None, :]
    c, s = torch.cos(a), torch.sin(a)
    out = x.clone()
    if neighbours:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., : dims // 2], x[..., dims // 2: dims]
        out[..., : dims // 2] = u * c - v * s
        out[..., dims // 2: dims] = v * c + u * s
    return out


# ----------------------------------------------------------------------------------- mixers
def decayed_sum_per_channel(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_a: torch.Tensor) -> torch.Tensor:
    """The recurrence S_t = diag(a_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t written as the explicit double sum
    o_t = sum_{s <= t} (sum_i q_t[i] k_s[i] prod_{s < r <= t} a_r[i]) v_s.   q, k, log_a [T, H, d], v [T, H, dv]."""
    T, H, _ = q.shape
    cum = log_a.cumsum(0)                                                     # log of the decay from the start to t
    o = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for t in range(T):
        wgt = torch.exp(cum[t][None] - cum[: t + 1])                          # [s, H, d]: prod_{s < r <= t} a_r
        score = (q[t][None] * k[: t + 1] * wgt).sum(-1)                       # [s, H]
        o[t] = torch.einsum("sh,shv->hv", score, v[: t + 1])
    return o


def decayed_sum_per_head(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay) -> torch.Tensor:
    """o_t = sum_{s <= t} g_h^(t - s) (q_t . k_s) v_s: the same recurrence with one fixed decay per head."""
    T, H, _ = q.shape
    t = torch.arange(T, dtype=q.dtype)
    dist = t[:, None] - t[None, :]
    o = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for hd in range(H):
        g = torch.tensor(float(decay[hd]), dtype=q.dtype)
        mask = torch.where(dist >= 0, g ** dist.clamp_min(0), torch.zeros((), dtype=q.dtype))
        o[:, hd] = ((q[:, hd] @ k[:, hd].T) * mask) @ v[:, hd]
    return o


def sigmoid_weighted_sum(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, temp: torch.Tensor,
                         bias: torch.Tensor) -> torch.Tensor:
    """o_i = sum_{j <= i} sigmoid((q_i . k_j) scale temp_h + bias_h) v_j; q [T, H, d], k [T, G, d], v [T, G, dv]."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    visible = torch.tril(torch.ones(T, T, dtype=torch.bool))
    o = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd // rep].T) * scale * temp[hd]
        o[:, hd] = (torch.sigmoid(s + bias[hd]) * visible) @ v[:, hd // rep]
    return o


def gated_linear_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, d)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    log_a = (torch.nn.functional.logsigmoid(z) / m["tau"]).view(T, H, d)
    o = unit_rms(decayed_sum_per_channel(q, k, v, log_a), m["eps"]) * w[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def sigmoid_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    """The values are the keys as projected: before their norm and rotation."""
    T = h.shape[0]
    H, G, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = (h @ w[p + "q"].T).view(T, H, d)
    k = (h @ w[p + "k"].T).view(T, G, d)
    qn = rotate_pairs(unit_rms(q, m["eps"]) * w[p + "q.norm"], rot["dims"], rot["base"], True)
    kn = rotate_pairs(unit_rms(k, m["eps"]) * w[p + "k.norm"], rot["dims"], rot["base"], True)
    o = sigmoid_weighted_sum(qn, kn, k, m["scale"], w[p + "temp"], w[p + "pb"])
    return o.reshape(T, H * d) @ w[p + "o"].T


def retention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_pairs((h @ w[p + "q"].T).view(T, H, d), rot["dims"], rot["base"], False)
    k = rotate_pairs((h @ w[p + "k"].T).view(T, H, d), rot["dims"], rot["base"], False) * d ** -0.5
    v = (h @ w[p + "v"].T).view(T, H, dv)
    o = unit_rms(decayed_sum_per_head(q, k, v, m["decay"]), m["eps"])
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


MIXERS = {"gla": gated_linear_attention, "attention": sigmoid_attention, "retention": retention}


# ----------------------------------------------------------------------------------- feed-forward
def route(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, r: dict):
    """Per token: the chosen experts and their weights, as lists of python numbers."""
    s = torch.sigmoid(h @ w[p + "router"].T)
    choice = s + w[p + "correction"]
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    gc, keep = groups["count"], groups["keep"]
    per = E // gc
    chosen, weights = [], []
    for t in range(h.shape[0]):
        c = choice[t].tolist()
        gscore = []
        for g in range(gc):
            members = sorted(c[g * per:(g + 1) * per], reverse=True)
            gscore.append(sum(members[:2]))
        best = sorted(range(gc), key=lambda g: (-gscore[g], g))[:keep]
        allowed = [e for e in range(E) if e // per in best]
        ids = sorted(allowed, key=lambda e: (-c[e], e))[:top]
        tot = sum(float(s[t, e]) for e in ids) + 1e-20
        chosen.append(ids)
        weights.append([float(s[t, e]) / tot * r.get("scale", 1.0) for e in ids])
    return chosen, weights


def mixture_of_experts(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    chosen, weights = route(h, w, p, mlp["router"])
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, c in zip(chosen[t], weights[t]):
            y[t] += c * (gelu_erf(h[t] @ w[f"{p}e{e}.up"].T) @ w[f"{p}e{e}.down"].T)
    return y


# ----------------------------------------------------------------------------------- side input
def token_side(x: torch.Tensor, tokens: List[int], w: Dict[str, torch.Tensor], layer: int, dim: int, eps: float) -> torch.Tensor:
    p = f"l{layer}.side."
    e = w["side.embed"][torch.tensor(tokens)][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w[p + "gate"].T) * e) @ w[p + "proj"].T
    return x + unit_rms(y, eps) * w[p + "norm"]


# ----------------------------------------------------------------------------------- the model
def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `streams`, if a list, receives the residual stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, groups, c = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["postln_alpha"]
    side = cfg.get("token_side")
    x = w["embed"][torch.tensor(tokens)]
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = dict(spec["mixer"], eps=eps)
        x = group_rms_norm(c * x + MIXERS[spec["type"]](x, w, p + "mix.", m), w[p + "norm1"], groups, eps)
        if spec.get("mlp") is not None:
            x = group_rms_norm(c * x + mixture_of_experts(x, w, p + "mlp.", spec["mlp"]), w[p + "norm2"], groups, eps)
        elif p + "norm2" in w:
            x = group_rms_norm(c * x, w[p + "norm2"], groups, eps)
        if side:
            x = token_side(x, tokens, w, i, side["dim"], eps)
        if streams is not None:
            streams.append(x.clone())
    return group_rms_norm(x, w["final.norm"], groups, eps) @ w["head"].T


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], n: int) -> List[int]:
    """n tokens generated greedily, every step a whole-sequence forward."""
    toks, out = list(tokens), []
    for _ in range(n):
        nxt = int(forward(cfg, weights, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
