"""Slow, plain implementation of the Kosalorn design, one function per
mechanism, written from the design's equations. It is the numerics oracle
of the tests: whole sequences at once, dense masks, float64, no cache, no
batching, keys and values decompressed per head — it shares no code with
the engine.

Notation: h is a layer's normed input [T, width]; W x means x @ W.T;
positions are 0..T-1.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return rms(x, eps) * g


def plain_norm(x, w, eps):
    """RMS norm with one weight per coordinate."""
    return rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate(x: torch.Tensor, base: float, dims: int, interleaved: bool) -> torch.Tensor:
    """Rotary positions on the first `dims` coordinates of the last axis of
    x [T, ..., n]; row t sits at position t. Pair i is (i, i + dims/2) in the
    half layout and (2i, 2i + 1) in the interleaved one; its angle is
    t * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = base ** (-2.0 * i / dims)
    ang = torch.arange(T, dtype=x.dtype).view(T, *([1] * (x.dim() - 2)), 1) * freq
    cos, sin = torch.cos(ang), torch.sin(ang)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


def visibility(T: int, window: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff j <= i and, with a window,
    i - j < window."""
    i = torch.arange(T).view(-1, 1)
    j = torch.arange(T).view(1, -1)
    vis = j <= i
    if window:
        vis = vis & (i - j < window)
    return vis


def latent_attention(h, w: Dict[str, torch.Tensor], cfg: dict, eps: float,
                     interleaved: bool) -> torch.Tensor:
    """Attention whose keys and values are expanded from a shared latent.
    With 'dq' tensors the query goes through a normed latent too."""
    T = h.shape[0]
    H, D, DR, DV, R = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    if "dq" in w:
        q = plain_norm(h @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T
    else:
        q = h @ w["q"].T
    q = q.view(T, H, D + DR)
    q_plain, q_rot = q[..., :D], q[..., D:]
    ckr = h @ w["dkv"].T
    c = plain_norm(ckr[:, :R], w["dkv.norm"], eps)
    k_rot = ckr[:, R:]                                  # [T, DR], one for all heads
    rot = cfg["rot"]
    q_rot = rotate(q_rot, rot["base"], rot["dims"], interleaved)
    k_rot = rotate(k_rot, rot["base"], rot["dims"], interleaved)
    k_plain = (c @ w["uk"].T).view(T, H, D)
    v = (c @ w["uv"].T).view(T, H, DV)
    scores = torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)
    scores = scores * cfg["scale"]
    window = cfg["mask"]["size"] if cfg.get("mask") else None
    scores = scores.masked_fill(~visibility(T, window).unsqueeze(0), float("-inf"))
    p = torch.softmax(scores, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v)
    return o.reshape(T, H * DV) @ w["o"].T


def hgrn2(h, w: Dict[str, torch.Tensor], cfg: dict, eps: float,
          state: Optional[torch.Tensor] = None):
    """Linear attention whose forget gate also sets the write strength.
    Token by token; returns (output, final state [H, D, DV])."""
    T = h.shape[0]
    H, D, DV = cfg["heads"], cfg["dim"], cfg["vdim"]
    q = silu(h @ w["q"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, DV)
    low = w["lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ w["f"].T + w["f.b"])).view(T, H, D)
    S = torch.zeros(H, D, DV, dtype=h.dtype) if state is None else state.clone()
    o = torch.empty(T, H, DV, dtype=h.dtype)
    for t in range(T):
        S = f[t].unsqueeze(-1) * S + (1.0 - f[t]).unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = plain_norm(o, w["norm"], eps)
    return o.reshape(T, H * DV) @ w["o"].T, S


def gated_ff(h, w: Dict[str, torch.Tensor], prefix: str = "") -> torch.Tensor:
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def expert_mixture(h, w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    """Each token feeds its `top` best-scoring experts with s * h, s the
    sigmoid of the router logit; the experts' outputs are summed."""
    E, top = cfg["router"]["experts"], cfg["router"]["top"]
    s = torch.sigmoid(h @ w["router"].T)                # [T, E]
    chosen = torch.topk(s, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += gated_ff((s[t, e] * h[t]).unsqueeze(0), w, f"e{e}.")[0]
    return out


def _sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_order(config: dict) -> List[tuple]:
    """[(layer index, adds the embedding output first)] in execution order."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for p in range(times):
        order += [(i, p > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def layer(x, tok, i: int, lc: dict, tw: Dict[str, torch.Tensor], config: dict):
    eps = config["norm"]["eps"]
    p = f"l{i}."
    h = scalar_norm(x, tw[p + "norm1"], eps)
    mw = _sub(tw, p + "mix.")
    if lc["type"] == "latent_attention":
        y = latent_attention(h, mw, lc["mixer"], eps, interleaved=False)
    elif lc["type"] == "latent_attention_2":
        y = latent_attention(h, mw, lc["mixer"], eps, interleaved=True)
    elif lc["type"] == "hgrn2":
        y, _ = hgrn2(h, mw, lc["mixer"], eps)
    else:
        raise ValueError(lc["type"])
    total = torch.sigmoid(h @ tw[p + "rg1"].T + tw[p + "rg1.b"]) * y
    mlp = lc.get("mlp")
    if mlp is not None:
        fw = _sub(tw, p + "mlp.")
        z = gated_ff(h, fw) if mlp["kind"] == "dense" else expert_mixture(h, fw, mlp)
        total = total + torch.sigmoid(h @ tw[p + "rg2"].T + tw[p + "rg2.b"]) * z
    x = x + total
    side = config.get("token_side")
    if side:
        d = side["dim"]
        e = tw["side.embed"][tok][:, i * d:(i + 1) * d]
        g = gelu_tanh(x @ tw[p + "side.gate"].T) * e
        x = x + plain_norm(g @ tw[p + "side.proj"].T, tw[p + "side.norm"], eps)
    return x


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int],
            dtype=F64, return_layers: bool = False):
    """Logits [T, vocab] for one whole sequence."""
    tw = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    x0 = scalar_norm(tw["embed"][tok], tw["embed.norm"], eps)
    x = x0
    runs = []
    for i, add_embedding in layer_order(config):
        if add_embedding:
            x = x + x0
        x = layer(x, tok, i, config["layers"][i], tw, config)
        runs.append(x)
    logits = scalar_norm(x, tw["final.norm"], eps) @ tw["head"].T
    if return_layers:
        return logits, torch.stack(runs)
    return logits


def greedy(config: dict, tensors: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """n greedy tokens after the prompt, recomputing the whole sequence each time."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, tensors, toks)[-1].argmax()))
    return toks[len(prompt):]
