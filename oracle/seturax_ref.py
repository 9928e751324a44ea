"""Plain, slow restatement of the Seturax design for checking the product path: one function per
mechanism, whole sequences at once, no cache, no batching, float64 by default.  Test infrastructure only;
nothing under sglang_custom_amd/ imports it and it imports nothing from there.

Notation: x [T, D] is the residual stream of ONE sequence, positions 0..T-1; weights come in a dict
under their checkpoint names (linear weights [out, in], applied as x @ W.T).

  embedding      x_t = E[tok_t] * s + B[(tok_{t-1} * m_prev + tok_t * m_cur) mod n]   (t = 0: B[n])
  layer          h = LN(x);  x <- x + sig(h Rg1 + b1) * mixer(shift(h)) + sig(h Rg2 + b2) * ff(h)
  shift          shift(h)_t = h_t + (h_{t-1} - h_t) * mu      (h_{-1} = 0)
  mixer          windowed multi-head attention whose keys and values are expanded from a shared latent,
                 with one extra term exp(sink_h) in every softmax denominator and a per-head sigmoid gate
  ff             down( gelu_tanh(gate h) * (up h) )
  output         logits = head LN(x) * logit_scale
"""
import json
import math
import os
import struct
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------------- file reading
def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """The safetensors container read by hand: u64 header length, JSON header, raw little-endian data."""
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32, "I64": torch.int64,
             "F64": torch.float64}
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        t = torch.frombuffer(bytearray(data[lo:hi]), dtype=kinds[meta["dtype"]])
        out[name] = t.reshape(meta["shape"]).clone()
    return out


def load_model(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ----------------------------------------------------------------------------------- small pieces
def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def embed(tokens: List[int], table: torch.Tensor, bigram: torch.Tensor, scale: float, mul_prev: int, mul_cur: int,
          buckets: int) -> torch.Tensor:
    rows = []
    for t, tok in enumerate(tokens):
        b = buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets
        rows.append(table[tok] * scale + bigram[b])
    return torch.stack(rows)


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def rotate_half(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, ..., n] with n >= dims: the first `dims` features are rotated (feature i pairs with i + dims/2),
    the rest pass through."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=v.dtype)
    a = positions.to(v.dtype)[:, None] * f[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = torch.cos(a).reshape(shape), torch.sin(a).reshape(shape)
    u, w = v[..., :half], v[..., half:dims]
    return torch.cat([u * c - w * s, w * c + u * s, v[..., dims:]], -1)


def window_mask(T: int, size: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j < size."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return ((i - j) >= 0) & ((i - j) < size)


def sink_softmax(scores: torch.Tensor, mask: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """scores [H, T, T], sink [H]: softmax over the visible keys with exp(sink_h) added to the denominator."""
    s = scores.masked_fill(~mask[None], float("-inf"))
    m = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - m))


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float) -> torch.Tensor:
    """h [T, D] -> [T, D].  p = '<layer>.mix.'"""
    T = h.shape[0]
    H, dn, dr, dv, rank = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    pos = torch.arange(T)
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(T, H, dn + dr)
    q_n, q_r = q[..., :dn], q[..., dn:]
    kv = h @ w[p + "dkv"].T
    c = rms_norm(kv[:, :rank], w[p + "dkv.norm"], eps)
    k_r = kv[:, rank:]                                       # [T, dr], shared by the heads
    k_n = (c @ w[p + "uk"].T).reshape(T, H, dn)
    v = (c @ w[p + "uv"].T).reshape(T, H, dv)
    rot = mx["rot"]
    q_r = rotate_half(q_r, pos, rot["base"], rot["dims"])
    k_r = rotate_half(k_r[:, None, :], pos, rot["base"], rot["dims"])[:, 0]
    scores = (torch.einsum("ihd,jhd->hij", q_n, k_n) + torch.einsum("ihd,jd->hij", q_r, k_r)) * mx["scale"]
    pr = sink_softmax(scores, window_mask(T, mx["mask"]["size"]), w[p + "sink"])
    o = torch.einsum("hij,jhd->ihd", pr, v)
    gate = torch.sigmoid(h @ w[p + "g"].T)                  # [T, H]
    o = o * gate[..., None]
    return o.reshape(T, H * dv) @ w[p + "o"].T


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def layer(x: torch.Tensor, w: Dict[str, torch.Tensor], i: int, spec: dict, eps: float) -> torch.Tensor:
    p = f"l{i}."
    h = layer_norm(x, w[p + "norm1"], eps)
    assert spec["type"] == "latent_attention"
    mix = latent_attention(token_shift(h, w[p + "shift"]), w, p + "mix.", spec["mixer"], eps)
    out = torch.sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"]) * mix
    if spec.get("mlp") is not None:
        assert spec["mlp"]["kind"] == "dense"
        out = out + torch.sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"]) * dense_ff(h, w, p + "mlp.")
    return x + out


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64, return_layers: bool = False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    e = cfg["embedding"]
    bg = e["bigram"]
    x = embed(tokens, w["embed"], w["bigram"], e["scale"], bg["mul_prev"], bg["mul_cur"], bg["buckets"])
    eps = cfg["norm"]["eps"]
    streams = []
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, w, i, spec, eps)
        streams.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["head"].T * cfg["logit_scale"]
    return (logits, torch.stack(streams)) if return_layers else logits


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], prompt: List[int], n: int, dtype=torch.float64) -> List[int]:
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks, dtype)[-1].argmax()))
    return toks[len(prompt):]


def absorbed_window_attention(qa: torch.Tensor, qr: torch.Tensor, c: torch.Tensor, kr: torch.Tensor, sink: torch.Tensor,
                              scale: float, window: int, base: float, dims: int, gate: Optional[torch.Tensor] = None,
                              first_position: int = 0) -> torch.Tensor:
    """The attention of latent_attention() with the key expansion folded into the query: qa [T, H, rank] multiplies
    the latent rows c [n, rank] directly, qr [T, H, dr] is the unrotated rope part, kr [n, dr] the ROTATED shared rope
    key of every cached position 0..n-1; the T queries sit at positions first_position .. first_position + T - 1
    (= n - 1).  Returns sum_j p_j c_j per head [T, H, rank], times sigmoid(gate [T, H]) if given."""
    T, n = qa.shape[0], c.shape[0]
    pos = torch.arange(first_position, first_position + T)
    q_rot = rotate_half(qr, pos, base, dims)
    scores = (torch.einsum("ihr,jr->hij", qa, c) + torch.einsum("ihd,jd->hij", q_rot, kr)) * scale
    mask = window_mask(n, window)[first_position: first_position + T]
    pr = sink_softmax(scores, mask, sink)
    o = torch.einsum("hij,jr->ihr", pr, c)
    return o if gate is None else o * torch.sigmoid(gate)[..., None]
