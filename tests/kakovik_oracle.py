"""Slow, plain implementation of the Kakovik design, one function per
mechanism, written from the design's equations. It is the numerics oracle
of the tests: whole sequences at once, dense masks, float64, no cache, no
batching — it shares no code with the engine.

Notation: h is a sublayer's normed input [T, width]; W x means x @ W.T.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def zero_centred_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * (1 + w)."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w)


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance-bias table for distance n >= 0: exact below
    rows/2, logarithmic up to `far`, clamped to the last row."""
    half = rows // 2
    if n < half:
        return n
    step = math.log(n / half) / math.log(far / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(step)))


def distance_bias(T: int, table: torch.Tensor, far: float) -> torch.Tensor:
    """[H, T, T] additive bias, entry (h, i, j) = table[bucket(i - j), h]
    for j <= i (0 above the diagonal, masked anyway)."""
    rows, H = table.shape
    per_dist = torch.stack([table[distance_bucket(n, rows, far)] for n in range(T)])  # [T, H]
    i = torch.arange(T).view(-1, 1)
    j = torch.arange(T).view(1, -1)
    return per_dist[(i - j).clamp(min=0)].permute(2, 0, 1).contiguous()


def block_causal_mask(T: int, size: int) -> torch.Tensor:
    """[T, T] bool, True where query i may see key j: j <= i and both in
    the same block of `size` positions counted from position 0."""
    i = torch.arange(T).view(-1, 1)
    j = torch.arange(T).view(1, -1)
    return (j <= i) & (i // size == j // size)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], cfg: dict,
                    eps: float, v_first: Optional[torch.Tensor]):
    """Returns (output [T, width], this layer's values before mixing)."""
    T = h.shape[0]
    H, G, D, DV = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = h @ w["q"].T
    k = h @ w["k"].T
    v = h @ w["v"].T
    # one norm over the whole projection, heads not yet split
    q = plain_rmsnorm(q, w["q.norm"], eps).view(T, H, D)
    k = plain_rmsnorm(k, w["k.norm"], eps).view(T, G, D)
    v_own = v
    if cfg.get("v_mix") and v_first is not None:
        lam = w["vmix"]
        v = (1.0 - lam) * v + lam * v_first
    v = v.view(T, G, DV)
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1)  # query head a uses kv head a // rep
    vh = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * cfg["scale"]
    scores = scores + distance_bias(T, w["rel"], cfg["bias_max"])
    mask = block_causal_mask(T, cfg["mask"]["size"])
    scores = scores.masked_fill(~mask.unsqueeze(0), float("-inf"))
    p = torch.softmax(scores, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, vh)  # [T, H, DV]
    gate = torch.sigmoid(h @ w["g"].T)  # [T, H]
    o = o * gate.unsqueeze(-1)
    return o.reshape(T, H * DV) @ w["o"].T, v_own


def gla_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], cfg: dict, eps: float,
              state: Optional[torch.Tensor] = None):
    """Gated linear attention, token by token. Returns (output, final state
    [H, D, DV])."""
    T = h.shape[0]
    H, D, DV, tau = cfg["heads"], cfg["dim"], cfg["vdim"], cfg["tau"]
    q = (h @ w["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, DV)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(T, H, D)
    S = torch.zeros(H, D, DV, dtype=h.dtype) if state is None else state.clone()
    o = torch.empty(T, H, DV, dtype=h.dtype)
    for t in range(T):
        S = alpha[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = plain_rmsnorm(o, w["norm"], eps)
    gate = torch.nn.functional.silu(h @ w["g"].T)
    return (o.reshape(T, H * DV) * gate) @ w["o"].T, S


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return (torch.nn.functional.silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def _sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int],
            dtype=F64, return_layers: bool = False):
    """Logits [T, vocab] for one whole sequence (positions 0..T-1)."""
    tw = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = tw["embed"][torch.tensor(tokens, dtype=torch.long)]
    v_first = None
    per_layer = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = zero_centred_rmsnorm(x, tw[p + "norm1"], eps)
        mw = _sub(tw, p + "mix.")
        if layer["type"] == "attention":
            mixes = bool(layer["mixer"].get("v_mix"))
            y, v_own = attention_mixer(h, mw, layer["mixer"], eps, v_first if mixes else None)
            if mixes and v_first is None:
                v_first = v_own
        elif layer["type"] == "gla":
            y, _ = gla_mixer(h, mw, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + zero_centred_rmsnorm(y, tw[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = zero_centred_rmsnorm(x, tw[p + "norm2"], eps)
            y = dense_ff(h, _sub(tw, p + "mlp."))
            x = x + zero_centred_rmsnorm(y, tw[p + "norm2b"], eps)
        per_layer.append(x)
    xf = zero_centred_rmsnorm(x, tw["final.norm"], eps)
    logits = xf @ tw["head"].T * config["logit_scale"]
    if return_layers:
        return logits, torch.stack(per_layer)
    return logits


def greedy(config: dict, tensors: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """n greedy tokens after the prompt, recomputing the whole sequence each time."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, tensors, toks)[-1].argmax()))
    return toks[len(prompt):]
