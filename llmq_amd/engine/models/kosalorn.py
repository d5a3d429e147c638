"""Kosalorn: a looped hybrid decoder on an fp32 residual.

A layer reads ONE norm (RMSNorm with a single-number weight) and feeds it to
a sequence mixer and a feed-forward in parallel; each result passes a sigmoid
gate computed from the same normed input before it joins the residual:

    h = norm(x);  x += sigmoid(W_g1 h + b1) * mixer(h) + sigmoid(W_g2 h + b2) * ff(h)

then a per-layer token-indexed side input is added:

    g = gelu_tanh(W_sg x) * side_embed[token, layer slice];  y = W_sp g
    x += rmsnorm(y) * w_side

Mixers: latent attention (keys and values expanded from a shared normed
latent, one rotated key part shared by all heads; with or without a query
latent; sliding-window or causal) and HGRN2 (a [dim, vdim] fp32 state per
head whose forget gate f = l + (1-l) sigmoid(.) also sets the write strength
1 - f). Feed-forwards: dense SiLU-gated, or a mixture of such experts picked
by sigmoid router scores that scale the expert's input. A range of layers may
run several times in a row with the same weights; every run owns its cache
or state, and every pass after the first starts by adding the embedding
output to the residual.

MI355X mapping, in the manner of the other families:

- plain-tensor weights; everything that reads h and is not a feed-forward is
  packed into ONE GEMM per layer (mixer input projections ‖ both gates);
- the residual stays fp32; the gated parallel join is one kernel that also
  hands the side-input GEMM its rounded copy, and the side input's norm,
  its residual add and the next layer's norm are one more;
- latent attention runs in the absorbed form: the query is mapped into the
  latent space (per-head W_uk^T q), attention runs directly over the cached
  [latent ‖ rotated key] rows shared by all heads, values are the rows'
  latent prefix, and W_uv is applied to the attended latent. The cache holds
  kv_rank + rot_dim numbers per token and layer run, nothing per head, and
  prompt portions and single tokens read it through the same block table;
- the HGRN2 state lives in per-sequence slots and is advanced by the same
  recurrence kernel as gated linear attention, in its lower-bounded mode;
- a step's expert mixture runs sorted by expert on vendor GEMMs, or, for few
  rows and inside captured decode graphs, as matrix-vector kernels that
  read only the chosen experts' weights.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Union

import torch
import torch.nn.functional as F

from llmq_amd import ops
from llmq_amd.engine.forward_meta import DecodeMeta, MixedMeta, PrefillMeta
from llmq_amd.engine.kv_cache import KVCache
from llmq_amd.engine.model_specs import KosalornSpec


def rotary_inv_freq(base: float, dims: int) -> torch.Tensor:
    """fp32 table base^(-2i/dims), i < dims/2, rounded once from float64."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * i / dims).to(torch.float32)


class KosalornLayerWeights:
    def __init__(self) -> None:
        self.t: Dict[str, torch.Tensor] = {}     # packed / checkpoint-shaped tensors
        self.seg: Dict[str, tuple] = {}          # name -> (first row, rows) in t["in"]
        self.norm_vec: Optional[torch.Tensor] = None   # the scalar norm weight, one per column
        self.inv_freq: Optional[torch.Tensor] = None   # fp32 rotary table (attention)


def _align8(n: int) -> int:
    return -(-n // 8) * 8


class KosalornLM:
    #: HIP extension groups this family runs on
    ext_groups = ("hybrid",)
    #: prompt portions attend through the block table (no gathered copy)
    paged_prefill = True
    #: mixed steps run their decode and prefill segments one after the other:
    #: this family's projection shapes select hipBLASLt stream-k GEMMs, whose
    #: workgroups wait on each other and must not share the chip with a second
    #: stream's kernels (LLMQ_OVERLAP_MIXED=1 forces the overlap back on)
    overlap_mixed = False

    def __init__(self, spec: KosalornSpec, device: torch.device, dtype: torch.dtype,
                 tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("the hybrid families run on one GPU per replica")
        self.spec = spec
        self.device = device
        self.dtype = dtype
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.runs = spec.runs()
        self.layers: List[KosalornLayerWeights] = []
        self.embedding: Optional[torch.Tensor] = None
        self.lm_head: Optional[torch.Tensor] = None
        self.side_embed: Optional[torch.Tensor] = None
        self.embed_norm = self._empty(())
        self.final_norm = self._empty(())
        self.embed_norm_vec: Optional[torch.Tensor] = None   # fp32 [W]
        self.final_norm_vec: Optional[torch.Tensor] = None   # dtype [W]
        self.taps: Optional[List[torch.Tensor]] = None  # residual after each layer run (debug)
        self._alloc()

    # -- layout the engine asks for: one entry per layer RUN ---------------

    def kv_layout(self):
        return [
            (1, self.spec.layers[i].mixer.kv_rank + self.spec.layers[i].mixer.rot_dim, 0)
            if self.spec.layers[i].mixer.kind == "latent_attention" else None
            for i, _ in self.runs
        ]

    def state_layout(self):
        out = []
        for i, _ in self.runs:
            m = self.spec.layers[i].mixer
            out.append((m.heads, m.dim, m.vdim) if m.kind == "hgrn2" else None)
        return out

    # -- weights ---------------------------------------------------------

    def _empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(*shape, device=self.device, dtype=dtype or self.dtype)

    def _alloc(self) -> None:
        s = self.spec
        W = s.hidden_size
        self.embedding = self._empty(s.vocab_size, W)
        self.lm_head = self._empty(s.vocab_size, W)
        if s.side_dim:
            self.side_embed = self._empty(s.vocab_size, s.side_dim * len(s.layers))
        for ls in s.layers:
            lw = KosalornLayerWeights()
            m, t = ls.mixer, lw.t
            t["norm1"] = self._empty(())
            # segments of the packed input projection, each starting at a
            # multiple of 8 rows (16-byte aligned column slices of its output)
            if m.kind == "hgrn2":
                nk, nv = m.heads * m.dim, m.heads * m.vdim
                segs = [("q", nk), ("f", nk), ("v", nv)]
                t["f_b"] = self._empty(nk, dtype=torch.float32)
                t["lower"] = self._empty(nk, dtype=torch.float32)
                t["norm"] = self._empty(m.vdim)
                t["o"] = self._empty(W, nv)
            else:
                nq = m.heads * (m.dim + m.rot_dim)
                if m.q_rank:
                    segs = [("dq", m.q_rank)]
                    t["dq_norm"] = self._empty(m.q_rank)
                    t["uq"] = self._empty(nq, m.q_rank)
                else:
                    segs = [("q", nq)]
                segs.append(("dkv", m.kv_rank + m.rot_dim))
                t["dkv_norm"] = self._empty(m.kv_rank)
                t["uk"] = self._empty(m.heads, m.dim, m.kv_rank)     # [H, dim, R]
                t["uv"] = self._empty(m.heads, m.vdim, m.kv_rank)    # [H, vdim, R]
                t["o"] = self._empty(W, m.heads * m.vdim)
            segs += [("rg1", W)]
            if ls.ff or ls.moe:
                segs += [("rg2", W)]
            at = 0
            for name, n in segs:
                lw.seg[name] = (at, n)
                at += _align8(n)
            t["in"] = self._empty(at, W)
            t["in"].zero_()
            t["rg1_b"] = self._empty(W, dtype=torch.float32)
            if ls.ff or ls.moe:
                t["rg2_b"] = self._empty(W, dtype=torch.float32)
            if ls.ff:
                t["gate_up"] = self._empty(2 * ls.ff, W)
                t["down"] = self._empty(W, ls.ff)
            if ls.moe:
                e = ls.moe
                t["router"] = self._empty(e.experts, W, dtype=torch.float32)
                t["e_gate_up"] = self._empty(e.experts, 2 * e.ff, W)
                t["e_down"] = self._empty(e.experts, W, e.ff)
            if s.side_dim:
                t["side_gate"] = self._empty(s.side_dim, W)
                t["side_proj"] = self._empty(W, s.side_dim)
                t["side_norm"] = self._empty(W)
            self.layers.append(lw)

    @torch.no_grad()
    def finalize(self) -> None:
        """Derive what the kernels read from the loaded tensors: the scalar
        norm weights as one value per column, and the rotary tables."""
        W = self.spec.hidden_size
        self.embed_norm_vec = self.embed_norm.float().expand(W).contiguous()
        self.final_norm_vec = self.final_norm.expand(W).contiguous()
        for ls, lw in zip(self.spec.layers, self.layers):
            lw.norm_vec = lw.t["norm1"].expand(W).contiguous()
            if ls.mixer.kind == "latent_attention":
                rot = ls.mixer.rot
                lw.inv_freq = rotary_inv_freq(rot.base, rot.dims).to(self.device)

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
        fill(self.embedding, 1.0)
        fill(self.lm_head, 1.0 / math.sqrt(W))
        if self.side_embed is not None:
            fill(self.side_embed, 1.0)
        self.embed_norm.fill_(1.0)
        self.final_norm.fill_(1.0)
        for lw in self.layers:
            for name, t in lw.t.items():
                if name == "norm1":
                    t.fill_(1.0)
                elif name in ("dq_norm", "dkv_norm", "norm", "side_norm"):
                    fill(t, 0.1, 1.0)
                elif name in ("rg1_b", "rg2_b", "f_b"):
                    fill(t, 0.5)
                elif name == "lower":
                    t.copy_(torch.rand(t.shape, generator=torch.Generator().manual_seed(seed))
                            .mul_(0.9).to(t.device))
                elif name == "in":
                    rows = t.shape[0]
                    fill(t, 1.0 / math.sqrt(W))
                    keep = torch.zeros(rows, dtype=torch.bool)
                    for at, n in lw.seg.values():
                        keep[at:at + n] = True
                    t[~keep.to(t.device)] = 0
                else:
                    fill(t, 1.0 / math.sqrt(t.shape[-1]))
        self.finalize()

    def named_tensors(self) -> Dict[str, torch.Tensor]:
        out = {"embedding": self.embedding, "lm_head": self.lm_head,
               "embed_norm": self.embed_norm, "final_norm": self.final_norm}
        if self.side_embed is not None:
            out["side_embed"] = self.side_embed
        for i, lw in enumerate(self.layers):
            for name, t in lw.t.items():
                out[f"layers.{i}.{name}"] = t
        return out

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.named_tensors().values())

    # -- mixers ----------------------------------------------------------

    def _seg(self, p: torch.Tensor, lw: KosalornLayerWeights, name: str) -> torch.Tensor:
        at, n = lw.seg[name]
        return p[:, at:at + n]

    def _latent_attention(self, p, lw, m, run, positions, kv_cache, meta):
        T = p.shape[0]
        H, D, DR, R = m.heads, m.dim, m.rot_dim, m.kv_rank
        eps = self.spec.rms_eps
        if m.q_rank:
            cq = ops.rmsnorm_cast(self._seg(p, lw, "dq"), lw.t["dq_norm"], eps, 0.0, self.dtype)
            q = F.linear(cq, lw.t["uq"])
        else:
            q = self._seg(p, lw, "q")
        q3 = q.view(T, H, D + DR) if q.is_contiguous() else q.unflatten(1, (H, D + DR))
        # the unrotated query part mapped into the latent space, per head
        q_lat = torch.bmm(q3[:, :, :D].transpose(0, 1), lw.t["uk"]).transpose(0, 1)  # [T, H, R]
        kc = kv_cache.k[run]
        qf = ops.latent_rope_pack(
            q3, q_lat, self._seg(p, lw, "dkv"), lw.t["dkv_norm"], lw.inv_freq, positions, kc,
            meta.slot_mapping, D, m.rot.dims, m.rot.layout == "interleaved", eps)
        if meta.is_prefill:
            ctx = ops.window_attn_prefill(
                qf, kc, None, R, meta.block_tables, meta.cu_seqlens, meta.q_start,
                meta.max_seqlen, m.window, m.scale)
        elif meta.is_mixed:
            nd, pm, dm = meta.n_decode, meta.prefill, meta.decode
            ctx_d = ops.window_attn_decode(
                qf[:nd], kc, None, R, dm.block_tables, dm.context_lens, m.window, m.scale)
            ctx_p = ops.window_attn_prefill(
                qf[nd:], kc, None, R, pm.block_tables, pm.cu_seqlens, pm.q_start,
                pm.max_seqlen, m.window, m.scale)
            ctx = torch.cat([ctx_d, ctx_p], dim=0)
        else:
            ctx = ops.window_attn_decode(
                qf, kc, None, R, meta.block_tables, meta.context_lens, m.window, m.scale)
        # values: W_uv on the attended latent, per head
        o = torch.bmm(ctx.transpose(0, 1), lw.t["uv"].transpose(1, 2))   # [H, T, vdim]
        return F.linear(o.transpose(0, 1).reshape(T, H * m.vdim), lw.t["o"])

    def _hgrn2(self, p, lw, m, run, kv_cache, meta):
        T = p.shape[0]
        q = self._seg(p, lw, "q").unflatten(1, (m.heads, m.dim))
        z = self._seg(p, lw, "f").unflatten(1, (m.heads, m.dim))
        v = self._seg(p, lw, "v").unflatten(1, (m.heads, m.vdim))
        rm = meta.recurrent
        o = ops.gated_recurrence(q, None, v, z, lw.t["f_b"], kv_cache.recurrent.state[run],
                                 rm.cu, rm.slots, rm.fresh, lower=lw.t["lower"], q_silu=True)
        y = ops.head_norm(o, lw.t["norm"], self.spec.rms_eps, self.dtype)
        return F.linear(y, lw.t["o"])

    def _moe(self, h, lw, e, meta):
        logits = F.linear(h.float(), lw.t["router"])
        idx, w = ops.sigmoid_topk(logits, e.top)
        decode_only = not (meta.is_prefill or meta.is_mixed)
        return ops.moe_experts(h, idx, w, lw.t["e_gate_up"], lw.t["e_down"],
                               sync_free=decode_only)

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
        emb = F.embedding(input_ids, self.embedding).float()
        res = ops.rmsnorm_cast(emb, self.embed_norm_vec, eps, 0.0, torch.float32)
        x0 = res.clone() if any(add for _, add in self.runs) else None
        n_runs = len(self.runs)
        first = self.layers[self.runs[0][0]].norm_vec if n_runs else self.final_norm_vec
        h = ops.rmsnorm_cast(res, first, eps, 0.0, self.dtype)
        for run, (i, _add) in enumerate(self.runs):
            ls, lw = s.layers[i], self.layers[i]
            m = ls.mixer
            p = F.linear(h, lw.t["in"])
            if m.kind == "hgrn2":
                y_mix = self._hgrn2(p, lw, m, run, kv_cache, meta)
            else:
                y_mix = self._latent_attention(p, lw, m, run, positions, kv_cache, meta)
            y_ff = g2 = b2 = None
            if ls.ff:
                act = ops.act_and_mul(F.linear(h, lw.t["gate_up"]), gelu=False)
                y_ff = F.linear(act, lw.t["down"])
            elif ls.moe:
                y_ff = self._moe(h, lw, ls.moe, meta)
            if y_ff is not None:
                g2, b2 = self._seg(p, lw, "rg2"), lw.t["rg2_b"]
            xb = ops.gated_residual_add(res, y_mix, self._seg(p, lw, "rg1"), lw.t["rg1_b"],
                                        y_ff, g2, b2, self.dtype)
            nxt = run + 1
            w_next = self.layers[self.runs[nxt][0]].norm_vec if nxt < n_runs else self.final_norm_vec
            adds_embedding = nxt < n_runs and self.runs[nxt][1]
            if s.side_dim:
                a = F.linear(xb, lw.t["side_gate"])
                g = ops.side_gate_mul(a, self.side_embed, input_ids, i * s.side_dim)
                y = F.linear(g, lw.t["side_proj"])
                h = ops.sandwich_norm_res32(y, res, lw.t["side_norm"], w_next, eps, 0.0)
                if self.taps is not None:
                    self.taps.append(res.clone())
                if adds_embedding:
                    res.add_(x0)
                    h = ops.rmsnorm_cast(res, w_next, eps, 0.0, self.dtype)
            else:
                if self.taps is not None:
                    self.taps.append(res.clone())
                if adds_embedding:
                    res.add_(x0)
                h = ops.rmsnorm_cast(res, w_next, eps, 0.0, self.dtype)
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [N, width] -> logits [N, vocab] fp32."""
        return F.linear(hidden, self.lm_head).float()
