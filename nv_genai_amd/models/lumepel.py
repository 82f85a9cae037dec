"""Lumepel decoder on the gfx950 kernel set: pre-norm layers on an fp32 residual stream, latent
attention with a rotated key part, clamped-GLU feed-forwards (dense or sigmoid-routed experts
with a gated shared expert), scaled and soft-capped logits.

Per layer (``x`` is the fp32 residual stream, activations in the model dtype):

    h  = norm1(x)                                  fused into the previous residual step
    x += mixer(h); h2 = norm2(x)                   ops.residual_add_rmsnorm_
    x += ff(h2);   h = next layer's norm1(x)       (same op)

Mixer (both kinds): one GEMM gives ``[q or query latent | latent | rotated key part]``;
``ops.latent_rope_cache_`` normalises the latent, rotates the shared key part, writes both into
the token's page slot (the only thing cached: ``kv_rank + rot_dim`` elements per token and
layer) and rotates the query heads' rotated parts. The attention runs in the latent space: the
key expansion is folded into the query (``(W_uk c) . q = c . (W_uk^T q)``), so a head's query is
``[W_uk^T q_unrotated | q_rotated]`` against the page row ``[c | k_rotated]``, the values are the
first ``kv_rank`` elements of the same row (``ops.softmax_attention(..., v_in_k=True)``:
multi-query attention, every head reads the one page), and the value expansion is applied to the
attention output. ``latent_attention`` sends the query through a normalised latent of its own
(a second GEMM) and pairs neighbouring elements in the rotation, with YaRN-scaled frequencies
when the config gives a scaling; ``latent_attention_2`` projects the query directly and pairs
element i with i + dims / 2.

Feed-forward: ``down(g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(gate h, limit)``,
``u = clamp(up h, -limit, limit)`` (``ops.clamped_glu``). Mixture layers route in fp32
(``sigmoid`` scores, the largest ``top``, not renormalised), put the routing weight on the
expert's *input* (``ops.moe_glu_experts``) and add a shared expert times ``sigmoid(sg . h)``.

The serving engine drives this class as it drives the other decoders (``forward`` on a step's token
rows + ``logits``); ``AttnMeta`` carries the per-step row maps (``tok_seq``).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..parallel.dist import ParallelContext, get_context
from .config import ClampedGluSpec, LumepelConfig, SigmoidMoeSpec
from .llama import AttnMeta

GLU_ALPHA = 1.702   # the sigmoid's slope in the gated activation: fixed by the design


def _ceil8(n: int) -> int:
    return (n + 7) // 8 * 8


class LumepelModel:
    stateful = True                # steps carry the engine's row maps (block-table row of every token)
    uses_decode_workspace = False
    supports_step_graphs = False   # prefill / mixed steps run eagerly (decode steps are graphs)
    supports_prefix_cache = True   # a page holds everything a token leaves behind

    def __init__(self, cfg: LumepelConfig, device="cuda", dtype=torch.bfloat16,
                 pctx: Optional[ParallelContext] = None, seed: int = 0,
                 weights: Optional[Dict[str, torch.Tensor]] = None, fp8: bool = False):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lumepel runs in bfloat16 or float32")
        if fp8:
            raise NotImplementedError("FP8 projections cover the Llama-layout decoders")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.p = pctx or get_context()
        if self.p.tp_size > 1 or self.p.pp_size > 1:
            raise NotImplementedError("Lumepel runs on one GPU per replica (no TP / PP split)")
        self.fp8 = False
        self.kv_dtype, self.kv_scales = "auto", (1.0, 1.0)
        self.sequence_parallel, self.sp_min_tokens, self.split_mixed, self.moe_ws = False, 0, False, None
        m0 = cfg.blocks[0].mixer
        self.hq, self.hkv, self.D = m0.heads, 1, m0.kv_rank + m0.rot_dim
        self.n_experts = cfg.num_experts
        self.vocab_local = cfg.vocab_size
        self.k_cache: List[Optional[torch.Tensor]] = []
        self.v_cache: List[Optional[torch.Tensor]] = []
        self.skinny = (self.device.type == "cuda" and dtype == torch.bfloat16 and ops.skinny.enabled())
        self.mfma = True   # MFMA attention / expert kernels where they apply (bf16, tile sizes)
        if weights is None:
            weights = random_weights(cfg, seed, dtype)
        self._load(weights)

    # ------------------------------------------------------------------ weights
    def _load(self, w: Dict[str, torch.Tensor]):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        H = cfg.hidden

        def mat(name, shape, dtype=dt):
            t = w[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, config says {tuple(shape)}")
            t = t.to(dev, dtype).contiguous()
            return t.clone() if t.data_ptr() % 16 else t   # (a memory-mapped file need not be aligned)

        def vec(name, n):
            t = w[name].to(dev, torch.float32).reshape(-1).contiguous()
            if t.numel() != n:
                raise ValueError(f"{name}: {t.numel()} elements, config says {n}")
            return t

        def fused(*mats):
            """Row-stacked GEMM weight, padded with zero rows to a multiple of 8 outputs."""
            W = torch.cat(mats)
            pad = _ceil8(W.shape[0]) - W.shape[0]
            if pad:
                W = torch.cat([W, torch.zeros(pad, W.shape[1], dtype=W.dtype, device=W.device)])
            return W.contiguous()

        def glu(p, s: ClampedGluSpec, extra=()):
            return (fused(mat(p + "gate", (s.ff, H)), mat(p + "up", (s.ff, H)), *extra), mat(p + "down", (H, s.ff)))

        self.embed = mat("embed", (cfg.vocab_size, H))
        self.layers: List[dict] = []
        for i, b in enumerate(cfg.blocks):
            p, m = f"l{i}.", b.mixer
            nq, r, dr = m.heads * (m.dim + m.rot_dim), m.kv_rank, m.rot_dim
            L = {"type": b.type, "spec": m, "mlp": b.mlp, "norm1": vec(p + "norm1", H)}
            dkv = mat(p + "mix.dkv", (r + dr, H))
            if m.q_rank:
                L["w_in"] = fused(mat(p + "mix.dq", (m.q_rank, H)), dkv)
                L["qn"] = vec(p + "mix.dq.norm", m.q_rank)
                L["wuq"] = fused(mat(p + "mix.uq", (nq, m.q_rank)))
                L["kv_off"] = m.q_rank
            else:
                L["w_in"] = fused(mat(p + "mix.q", (nq, H)), dkv)
                L["kv_off"] = nq
            L["cn"] = vec(p + "mix.dkv.norm", r)
            freq, mag = ops.rotary_frequencies(m.rot.dims, m.rot.base, m.rot.yarn)
            L["freq"], L["mag"] = freq.to(dev), mag
            # per head: W_uk [dim, r] folds into the query, W_uv^T [r, vdim] expands the output
            L["wuk"] = mat(p + "mix.uk", (m.heads * m.dim, r)).view(m.heads, m.dim, r).contiguous()
            L["wuvT"] = mat(p + "mix.uv", (m.heads * m.vdim, r)).view(m.heads, m.vdim, r).transpose(1, 2).contiguous()
            L["wo"] = mat(p + "mix.o", (H, m.heads * m.vdim))
            f = b.mlp
            if f is not None:
                L["norm2"] = vec(p + "norm2", H)
            if isinstance(f, SigmoidMoeSpec):
                L["router"] = mat(p + "mlp.router", (f.experts, H), torch.float32)
                ex = [glu(f"{p}mlp.e{e}.", f.expert) for e in range(f.experts)]
                L["w13"] = torch.stack([g[:2 * f.expert.ff] for g, _ in ex]).contiguous()
                L["w2"] = torch.stack([d for _, d in ex]).contiguous()
                if f.shared is not None:
                    L["wsgu"], L["wsd"] = glu(p + "mlp.shared.", f.shared, (mat(p + "mlp.shared.sg", (1, H)),))
            elif f is not None:
                L["wgu"], L["wd"] = glu(p + "mlp.", f)
            self.layers.append(L)
        self.final_norm = vec("final.norm", H)
        self.lm_head = mat("head", (cfg.vocab_size, H))

    def state_dict(self) -> Dict[str, torch.Tensor]:
        dt, H = self.dtype, self.cfg.hidden
        out = {"embed": self.embed, "final.norm": self.final_norm.to(dt), "head": self.lm_head}
        for i, L in enumerate(self.layers):
            p, m, f = f"l{i}.", L["spec"], L["mlp"]
            nq, r, dr = m.heads * (m.dim + m.rot_dim), m.kv_rank, m.rot_dim
            out[p + "norm1"] = L["norm1"].to(dt)
            W, o = L["w_in"], L["kv_off"]
            if m.q_rank:
                out.update({p + "mix.dq": W[:o], p + "mix.dq.norm": L["qn"].to(dt), p + "mix.uq": L["wuq"][:nq]})
            else:
                out[p + "mix.q"] = W[:o]
            out.update({p + "mix.dkv": W[o:o + r + dr], p + "mix.dkv.norm": L["cn"].to(dt),
                        p + "mix.uk": L["wuk"].reshape(m.heads * m.dim, r),
                        p + "mix.uv": L["wuvT"].transpose(1, 2).reshape(m.heads * m.vdim, r), p + "mix.o": L["wo"]})
            if f is not None:
                out[p + "norm2"] = L["norm2"].to(dt)
            if isinstance(f, SigmoidMoeSpec):
                F = f.expert.ff
                out[p + "mlp.router"] = L["router"].to(dt)
                for e in range(f.experts):
                    out.update({f"{p}mlp.e{e}.gate": L["w13"][e, :F], f"{p}mlp.e{e}.up": L["w13"][e, F:],
                                f"{p}mlp.e{e}.down": L["w2"][e]})
                if f.shared is not None:
                    Fs = f.shared.ff
                    out.update({p + "mlp.shared.gate": L["wsgu"][:Fs], p + "mlp.shared.up": L["wsgu"][Fs:2 * Fs],
                                p + "mlp.shared.sg": L["wsgu"][2 * Fs:2 * Fs + 1], p + "mlp.shared.down": L["wsd"]})
            elif f is not None:
                out.update({p + "mlp.gate": L["wgu"][:f.ff], p + "mlp.up": L["wgu"][f.ff:2 * f.ff], p + "mlp.down": L["wd"]})
        return out

    # ------------------------------------------------------------------ cache
    def allocate_kv_cache(self, num_blocks: int, block_size: int = 64, kv_dtype: str = "auto",
                          kv_scales=(1.0, 1.0)):
        """One page tensor per layer, [blocks, 1, 64, kv_rank + rot_dim] in the model dtype: a
        token's row is its normalised latent followed by the rotated key part. The attention
        kernels read the row as the key and its first kv_rank elements as the value. All layers
        are addressed by the same page numbers."""
        if block_size != 64:
            raise ValueError("the gfx950 attention kernels use 64-token KV pages")
        if kv_dtype not in ("auto", "bf16"):
            raise ValueError("Lumepel keeps its pages in the model dtype")
        self.k_cache = [torch.zeros(num_blocks, 1, block_size, L["spec"].kv_rank + L["spec"].rot_dim,
                                    device=self.device, dtype=self.dtype) for L in self.layers]
        self.v_cache = list(self.k_cache)
        return self.k_cache, self.v_cache

    def allocate_state(self, slots: int) -> None:
        """Nothing besides the pages is carried from step to step."""

    def kv_block_bytes(self, block_size: int = 64, kv_dtype: str = "auto") -> int:
        elem = torch.finfo(self.dtype).bits // 8
        return sum(b.mixer.kv_rank + b.mixer.rot_dim for b in self.cfg.blocks) * block_size * elem

    def copy_kv_blocks(self, src, dst) -> None:
        for c in self.k_cache:
            c[dst] = c[src]

    def ipc_collectives_cover(self, rows: int, tokens: int) -> bool:
        return True

    def quantize_fp8(self) -> None:
        raise NotImplementedError("FP8 projections cover the Llama-layout decoders")

    # ------------------------------------------------------------------ forward
    def _lin(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w^T: decode-shape rows take the skinny MFMA GEMM where the measured table
        (ops.skinny) holds this (N, K) and prefers it over the library GEMM."""
        if self.skinny and x.shape[0] <= 512 and x.stride(1) == 1 and x.stride(0) % 8 == 0:
            pk = ops.skinny.table().pick(w.shape[0], w.shape[1], x.shape[0])
            if pk is not None:
                cfg, split = pk
                if split == 1:
                    return ops.skinny_gemm(x, w, cfg, 1, 0)
                return ops.PartialSum(ops.skinny_gemm(x, w, cfg, split, 1)).materialize()
        return ops.linear(x, w)

    def _attend(self, q, page, pos, meta: AttnMeta, H, dk, dv, scale):
        """Multi-query softmax attention of a step's rows over the latent page (values inside
        the key rows): prompt portions on the MFMA tile kernel and single-token rows on the
        page-parallel kernel where they apply (bf16, tile sizes), everything else on the row
        kernel."""
        kw = dict(scale=scale, window=0, v_in_k=True)
        if self.mfma and ops.softmax_attention_mfma_ok(q, dk, dv, H, 1):
            nd = meta.n_decode if meta.kind == "mixed" else (q.shape[0] if meta.kind == "decode" else 0)
            out = torch.empty(q.shape[0], H * dv, dtype=q.dtype, device=q.device)
            if nd:
                ops.softmax_attention_rows(q[:nd], page, page, meta.block_tables, meta.tok_seq[:nd], pos[:nd], H, 1,
                                           dk, dv, max_ctx=meta.max_ctx, out=out[:nd], **kw)
            if nd < q.shape[0]:
                ops.softmax_attention_prefill(q[nd:], page, page, meta.block_tables[nd:],
                                              meta.cu_q_prefill if nd else meta.cu_q, meta.ctx_lens[nd:],
                                              meta.max_q_len, H, 1, dk, dv, out=out[nd:], **kw)
            return out
        return ops.softmax_attention(q, page, page, meta.block_tables, meta.tok_seq, pos, H, 1, dk, dv, **kw)

    def _mixer(self, li: int, h, pos, meta: AttnMeta):
        L = self.layers[li]
        m = L["spec"]
        T, Hh, d, dr, r = h.shape[0], m.heads, m.dim, m.rot_dim, m.kv_rank
        W = r + dr
        page = self.k_cache[li]
        rope = (L["freq"], L["mag"], m.rot.interleaved, m.rot.dims, dr, self.cfg.eps)
        proj = self._lin(h, L["w_in"])
        qf = torch.empty(T, Hh * W, dtype=h.dtype, device=h.device)
        kv = (L["kv_off"], r, L["cn"])
        if m.q_rank:
            ops.latent_rope_cache_(proj, pos, meta.slots, page, *rope, kv=kv, norm=(0, m.q_rank, L["qn"]))
            qp = self._lin(proj[:, :m.q_rank], L["wuq"])
            ops.latent_rope_cache_(qp, pos, meta.slots, None, *rope, q=(0, Hh, d), q_out=qf)
        else:
            qp = proj
            ops.latent_rope_cache_(proj, pos, meta.slots, page, *rope, kv=kv, q=(0, Hh, d), q_out=qf)
        qn = qp[:, :Hh * (d + dr)].view(T, Hh, d + dr)[:, :, :d].transpose(0, 1)      # [H, T, dim] view
        qf.view(T, Hh, W)[:, :, :r].copy_(torch.bmm(qn, L["wuk"]).transpose(0, 1))
        a = self._attend(qf, page, pos, meta, Hh, W, r, m.scale)
        av = torch.bmm(a.view(T, Hh, r).transpose(0, 1), L["wuvT"])                   # [H, T, vdim]
        return self._lin(av.transpose(0, 1).reshape(T, Hh * m.vdim), L["wo"])

    def _glu(self, h, wgu, wd, s: ClampedGluSpec, gate_col: int = -1):
        return self._lin(ops.clamped_glu(self._lin(h, wgu), s.ff, s.limit, GLU_ALPHA, gate_col), wd)

    def _ff(self, li: int, h):
        L = self.layers[li]
        f = L["mlp"]
        if not isinstance(f, SigmoidMoeSpec):
            return self._glu(h, L["wgu"], L["wd"], f)
        logits = ops.linear(h if h.dtype == torch.float32 else h.float(), L["router"])
        ids, wts = ops.moe_route_scores(logits, f.top, "sigmoid", False, ws=self.moe_ws)
        shared = None
        if f.shared is not None:
            shared = self._glu(h, L["wsgu"], L["wsd"], f.shared, gate_col=2 * f.shared.ff)
        return ops.moe_glu_experts(h, ids, wts, L["w13"], L["w2"], f.expert.limit, GLU_ALPHA, weight_input=True,
                                   add=shared, ws=self.moe_ws)

    def forward(self, ids: torch.Tensor, pos: torch.Tensor, meta: AttnMeta,
                sample_idx: Optional[torch.Tensor] = None, embed_override=None,
                layer_tap: Optional[list] = None) -> torch.Tensor:
        """Final-normed rows selected by ``sample_idx`` (all rows if None) of a step's token rows.
        ``layer_tap``: a list that receives a copy of the residual stream after every layer."""
        if embed_override is not None:
            raise NotImplementedError("Lumepel takes token ids only")
        if meta.tok_seq is None:
            raise ValueError("Lumepel steps need the engine's row maps (tok_seq)")
        eps, dt = self.cfg.eps, self.dtype
        x = ops.embed_rows(ids, self.embed, self.cfg.embed_scale)
        h = ops.rmsnorm_f32(x, self.layers[0]["norm1"], eps, dtype=dt)
        n = len(self.layers)
        for li, L in enumerate(self.layers):
            y = self._mixer(li, h, pos, meta)
            if L["mlp"] is not None:
                h2 = ops.residual_add_rmsnorm_(x, y, L["norm2"], eps, dt)
                y = self._ff(li, h2)
            h = ops.residual_add_rmsnorm_(x, y, self.layers[li + 1]["norm1"] if li + 1 < n else None, eps, dt)
            if layer_tap is not None:
                layer_tap.append(x.clone())
        return ops.rmsnorm_f32(x, self.final_norm, eps, rows=sample_idx, dtype=dt)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        z = ops.linear(h, self.lm_head).float()
        return ops.scale_softcap_(z, self.cfg.logit_scale, self.cfg.logit_softcap)


def random_weights(cfg: LumepelConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random weights under the checkpoint's tensor names (benchmarks, tests, smoke runs)."""
    g = torch.Generator().manual_seed(seed)
    H = cfg.hidden

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    def around1(n):
        return (1.0 + 0.1 * torch.randn(n, generator=g)).to(dtype)

    def glu(p, s: ClampedGluSpec, std_in=H ** -0.5):
        return {p + "gate": rnd(s.ff, H, std=std_in), p + "up": rnd(s.ff, H, std=std_in),
                p + "down": rnd(H, s.ff, std=s.ff ** -0.5)}

    w = {"embed": rnd(cfg.vocab_size, H, std=1.0), "final.norm": around1(H), "head": rnd(cfg.vocab_size, H, std=H ** -0.5)}
    s = H ** -0.5
    for i, b in enumerate(cfg.blocks):
        p, m = f"l{i}.", b.mixer
        nq, r, dr = m.heads * (m.dim + m.rot_dim), m.kv_rank, m.rot_dim
        w[p + "norm1"] = around1(H)
        if m.q_rank:
            w.update({p + "mix.dq": rnd(m.q_rank, H, std=s), p + "mix.dq.norm": around1(m.q_rank),
                      p + "mix.uq": rnd(nq, m.q_rank, std=m.q_rank ** -0.5)})
        else:
            w[p + "mix.q"] = rnd(nq, H, std=s)
        w.update({p + "mix.dkv": rnd(r + dr, H, std=s), p + "mix.dkv.norm": around1(r),
                  p + "mix.uk": rnd(m.heads * m.dim, r, std=r ** -0.5),
                  p + "mix.uv": rnd(m.heads * m.vdim, r, std=r ** -0.5),
                  p + "mix.o": rnd(H, m.heads * m.vdim, std=(m.heads * m.vdim) ** -0.5)})
        f = b.mlp
        if f is not None:
            w[p + "norm2"] = around1(H)
        if isinstance(f, SigmoidMoeSpec):
            w[p + "mlp.router"] = rnd(f.experts, H, std=s)
            for e in range(f.experts):
                w.update(glu(f"{p}mlp.e{e}.", f.expert))
            if f.shared is not None:
                w.update(glu(p + "mlp.shared.", f.shared))
                w[p + "mlp.shared.sg"] = rnd(1, H, std=s)
        elif f is not None:
            w.update(glu(p + "mlp.", f))
    return w
