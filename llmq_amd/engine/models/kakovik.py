"""Kakovik: a hybrid decoder — per-layer sequence mixers on an fp32 residual.

Layer i:  x += norm_b(mixer(norm(x)));  x += norm_b(ff(norm(x)))  (ff optional)
with zero-centred RMSNorm weights (1 + w). Mixers:

- block-local attention: keys limited to the query's span of positions, a
  learned bias per bucketed distance instead of a rotation, one RMSNorm over
  the whole q / k projection, value blending with the first blending layer's
  values, a sigmoid gate per head;
- gated linear attention: a [dim, vdim] fp32 state per head and sequence,
  decayed per key channel.

MI355X mapping, in the manner of the other families:

- plain-tensor weights, projections packed so each sublayer opens with ONE
  GEMM: attention q‖k‖v‖gate, GLA q‖k‖v‖gate‖decay-inner, ff gate‖up;
- the residual stays fp32 end to end; every sublayer boundary is one fused
  kernel (post-norm + residual add + next pre-norm, ops.sandwich_norm_res32);
- attention reads keys and values through the block table in BOTH the
  prompt-portion and the single-token kernel (the portion's rows are
  scattered into the paged cache first, fused with the q/k norms), so where
  a prompt is cut cannot change what a position sees;
- the GLA state lives in per-sequence slots (RecurrentStateCache) and is
  advanced by one kernel for any mix of portions and single tokens.

The per-distance bias is tabulated once per layer for distances inside one
span (bias[h, n], n < span) — the kernels index it by i - j.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Union

import torch
import torch.nn.functional as F

from llmq_amd import ops
from llmq_amd.engine.forward_meta import DecodeMeta, MixedMeta, PrefillMeta
from llmq_amd.engine.kv_cache import KVCache
from llmq_amd.engine.model_specs import HybridSpec


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Bias-table row of distance n: identity below rows/2, then log-spaced
    so that distance `far` reaches the last row; clamped there."""
    half = rows // 2
    if n < half:
        return n
    r = half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))
    return min(rows - 1, r)


class HybridLayerWeights:
    def __init__(self) -> None:
        self.t: Dict[str, torch.Tensor] = {}   # checkpoint-shaped tensors
        self.bias: Optional[torch.Tensor] = None   # [H, span] fp32 (attention)
        self.lam: float = 0.0                      # value-blend weight
        self.mixes: bool = False                   # blends with v_first
        self.provides_v_first: bool = False


class KakovikLM:
    #: HIP extension groups this family runs on
    ext_groups = ("hybrid",)
    #: prompt portions attend through the block table (no gathered copy)
    paged_prefill = True

    def __init__(self, spec: HybridSpec, device: torch.device, dtype: torch.dtype,
                 tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("the hybrid family runs on one GPU per replica")
        self.spec = spec
        self.device = device
        self.dtype = dtype
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.layers: List[HybridLayerWeights] = []
        self.embedding: Optional[torch.Tensor] = None
        self.final_norm: Optional[torch.Tensor] = None
        self.lm_head: Optional[torch.Tensor] = None
        self.taps: Optional[List[torch.Tensor]] = None  # residual after each layer (debug)
        self._alloc()

    # -- layout the engine asks for -------------------------------------

    def kv_layout(self):
        return [
            (ls.mixer.kv_heads, ls.mixer.dim, ls.mixer.vdim)
            if ls.mixer.kind == "attention" else None
            for ls in self.spec.layers
        ]

    def state_layout(self):
        return [
            (ls.mixer.heads, ls.mixer.dim, ls.mixer.vdim)
            if ls.mixer.kind == "gla" else None
            for ls in self.spec.layers
        ]

    # -- weights ---------------------------------------------------------

    def _empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(*shape, device=self.device, dtype=dtype or self.dtype)

    def _alloc(self) -> None:
        s = self.spec
        W = s.hidden_size
        self.embedding = self._empty(s.vocab_size, W)
        self.lm_head = self._empty(s.vocab_size, W)
        self.final_norm = self._empty(W)
        first_mix = True
        for ls in s.layers:
            lw = HybridLayerWeights()
            m = ls.mixer
            t = lw.t
            t["norm1"], t["norm1b"] = self._empty(W), self._empty(W)
            if m.kind == "attention":
                nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
                if m.heads % m.kv_heads:
                    raise ValueError("heads must be a multiple of kv_heads")
                # rows padded to a multiple of 8: row strides of the GEMM
                # output stay 16-byte aligned for the vector loads of q
                t["qkvg"] = self._empty(-(-(nq + nk + nv + m.heads) // 8) * 8, W)
                t["qkvg"].zero_()
                t["q_norm"], t["k_norm"] = self._empty(nq), self._empty(nk)
                t["rel"] = self._empty(m.bias_rows, m.heads)
                t["vmix"] = self._empty(())
                t["o"] = self._empty(W, m.heads * m.vdim)
                if m.v_mix:
                    lw.provides_v_first = first_mix
                    lw.mixes = not first_mix
                    first_mix = False
            else:
                nk, nv = m.heads * m.dim, m.heads * m.vdim
                t["qkvga"] = self._empty(2 * nk + 2 * nv + m.decay_rank, W)
                t["a2"] = self._empty(nk, m.decay_rank)
                t["a2_b"] = self._empty(nk, dtype=torch.float32)
                t["norm"] = self._empty(m.vdim)
                t["o"] = self._empty(W, nv)
            if ls.ff:
                t["norm2"], t["norm2b"] = self._empty(W), self._empty(W)
                t["gate_up"] = self._empty(2 * ls.ff, W)
                t["down"] = self._empty(W, ls.ff)
            self.layers.append(lw)

    @torch.no_grad()
    def finalize(self) -> None:
        """Derive what the kernels read from the loaded tensors: the
        per-distance bias table and the blend weight of each layer."""
        nv_first = None
        for ls, lw in zip(self.spec.layers, self.layers):
            m = ls.mixer
            if m.kind != "attention":
                continue
            rel = lw.t["rel"].float().cpu()
            # distances inside one span, and never beyond the longest context
            n_dist = min(m.span, self.spec.max_position_embeddings)
            rows = [distance_bucket(n, m.bias_rows, m.bias_far) for n in range(n_dist)]
            lw.bias = rel[torch.tensor(rows, dtype=torch.long)].t().contiguous().to(self.device)
            lw.lam = float(lw.t["vmix"].float().item())
            if m.v_mix:
                nv = m.kv_heads * m.vdim
                if nv_first is None:
                    nv_first = nv
                elif nv != nv_first:
                    raise ValueError("value-blending layers must share the value width")

    @torch.no_grad()
    def random_init(self, seed: int = 0, fast: bool = False) -> None:
        if fast and self.device.type == "cuda":
            gen = torch.Generator(device=self.device).manual_seed(seed)

            def fill(t: torch.Tensor, std: float, mean: float = 0.0) -> None:
                t.normal_(mean, std, generator=gen)
        else:
            gen = torch.Generator(device="cpu").manual_seed(seed)

            def fill(t: torch.Tensor, std: float, mean: float = 0.0) -> None:
                cpu = torch.randn(t.shape, generator=gen, dtype=torch.float32) * std + mean
                t.copy_(cpu.to(t.dtype))

        W = self.spec.hidden_size
        std = 1.0 / math.sqrt(W)
        fill(self.embedding, 1.0)
        fill(self.lm_head, std)
        fill(self.final_norm, 0.1)
        for ls, lw in zip(self.spec.layers, self.layers):
            for name, t in lw.t.items():
                if name.startswith("norm") or name in ("q_norm", "k_norm"):
                    fill(t, 0.1, 1.0 if name in ("q_norm", "k_norm", "norm") else 0.0)
                elif name == "rel":
                    fill(t, 0.5)
                elif name == "vmix":
                    t.fill_(0.3)
                elif name == "a2_b":
                    fill(t, 0.5, 2.0)
                else:
                    fill(t, 1.0 / math.sqrt(t.shape[-1]))
        self.finalize()

    def named_tensors(self) -> Dict[str, torch.Tensor]:
        out = {"embedding": self.embedding, "final_norm": self.final_norm,
               "lm_head": self.lm_head}
        for i, lw in enumerate(self.layers):
            for name, t in lw.t.items():
                out[f"layers.{i}.{name}"] = t
        return out

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.named_tensors().values())

    # -- mixers ----------------------------------------------------------

    def _attention(self, h, lw, m, i, kv_cache, meta, v_first):
        T = h.shape[0]
        nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        p = F.linear(h, lw.t["qkvg"])
        q, k, v = p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:nq + nk + nv]
        gate = p[:, nq + nk + nv:nq + nk + nv + m.heads]
        kc, vc = kv_cache.k[i], kv_cache.v[i]
        ops.qknorm_vmix_cache(
            q, k, v, lw.t["q_norm"], lw.t["k_norm"],
            v_first if lw.mixes else None, lw.lam, kc, vc, meta.slot_mapping,
            self.spec.rms_eps,
        )
        q3 = q.view(T, m.heads, m.dim)
        if meta.is_prefill:
            att = ops.chunk_bias_attn_prefill(
                q3, gate, kc, vc, lw.bias, meta.block_tables, meta.cu_seqlens,
                meta.q_start, meta.max_seqlen, m.span, m.scale)
        elif meta.is_mixed:
            nd, pm, dm = meta.n_decode, meta.prefill, meta.decode
            att_d = ops.chunk_bias_attn_decode(
                q3[:nd], gate[:nd], kc, vc, lw.bias, dm.block_tables, dm.context_lens,
                m.span, m.scale)
            att_p = ops.chunk_bias_attn_prefill(
                q3[nd:], gate[nd:], kc, vc, lw.bias, pm.block_tables, pm.cu_seqlens,
                pm.q_start, pm.max_seqlen, m.span, m.scale)
            att = torch.cat([att_d, att_p], dim=0)
        else:
            att = ops.chunk_bias_attn_decode(
                q3, gate, kc, vc, lw.bias, meta.block_tables, meta.context_lens,
                m.span, m.scale)
        return F.linear(att.view(T, m.heads * m.vdim), lw.t["o"]), v

    def _gla(self, h, lw, m, i, kv_cache, meta):
        T = h.shape[0]
        nk, nv = m.heads * m.dim, m.heads * m.vdim
        p = F.linear(h, lw.t["qkvga"])
        q = p[:, :nk].view(T, m.heads, m.dim)
        k = p[:, nk:2 * nk].view(T, m.heads, m.dim)
        v = p[:, 2 * nk:2 * nk + nv].view(T, m.heads, m.vdim)
        gate = p[:, 2 * nk + nv:2 * nk + 2 * nv]
        z = F.linear(p[:, 2 * nk + 2 * nv:], lw.t["a2"]).view(T, m.heads, m.dim)
        rm = meta.recurrent
        o = ops.gla_recurrence(q, k, v, z, lw.t["a2_b"], kv_cache.recurrent.state[i],
                               rm.cu, rm.slots, rm.fresh, m.tau)
        y = ops.gla_out_norm_gate(o, lw.t["norm"], gate, self.spec.rms_eps, self.dtype)
        return F.linear(y, lw.t["o"])

    # -- forward ---------------------------------------------------------

    @torch.no_grad()
    def forward(
        self,
        input_ids: torch.Tensor,
        positions: torch.Tensor,
        kv_cache: KVCache,
        meta: Union[PrefillMeta, DecodeMeta, MixedMeta],
    ) -> torch.Tensor:
        s = self.spec
        eps = s.rms_eps
        res = F.embedding(input_ids, self.embedding).float()
        n = len(self.layers)
        h = ops.rmsnorm_cast(res, self.layers[0].t["norm1"], eps, 1.0, self.dtype) if n else None
        v_first = None
        for i, (ls, lw) in enumerate(zip(s.layers, self.layers)):
            m = ls.mixer
            if m.kind == "attention":
                y, v_own = self._attention(h, lw, m, i, kv_cache, meta, v_first)
                if lw.provides_v_first:
                    v_first = v_own
            else:
                y = self._gla(h, lw, m, i, kv_cache, meta)
            w_next = self.layers[i + 1].t["norm1"] if i + 1 < n else self.final_norm
            h = ops.sandwich_norm_res32(
                y, res, lw.t["norm1b"], lw.t["norm2"] if ls.ff else w_next, eps, 1.0)
            if ls.ff:
                act = ops.act_and_mul(F.linear(h, lw.t["gate_up"]), gelu=False)
                y = F.linear(act, lw.t["down"])
                h = ops.sandwich_norm_res32(y, res, lw.t["norm2b"], w_next, eps, 1.0)
            if self.taps is not None:
                self.taps.append(res.clone())
        if n == 0:
            h = ops.rmsnorm_cast(res, self.final_norm, eps, 1.0, self.dtype)
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [N, width] → logits [N, vocab] fp32."""
        return F.linear(hidden, self.lm_head).float() * self.spec.logit_scale
