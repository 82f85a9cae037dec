"""Lizezen decoder on the gfx950 kernel set: parallel layers behind one dynamic-tanh norm on an
fp32 residual stream, mLSTM and rotary softmax-attention mixers, GELU or routed SwiGLU
feed-forwards, and a span of layers that runs several times with an input injection in front of
every pass.

Per layer run (``x`` is the fp32 residual stream, activations in the model dtype):

    h  = tanh(alpha x) * w + b                     fused into the previous residual step
    x += mixer(h) + ff(h); h = next run's norm     ops.residual_dyt_ (one launch)

In front of every pass of the repeated span the stream becomes ``W_in [x ; x0]`` (x0 = the
embedding rows): ``ops.pack_pair`` + one GEMM + ``ops.residual_dyt_(assign=True)``. Every layer
*run* has pages / a state slot tensor of its own, so the passes of the span do not share a cache.

Mixers:

* ``mlstm`` - one GEMM gives ``q | k | v | output gate | i | f``; ``ops.mlstm_scan`` carries the
  fp32 state (S, n, m) of every sequence in a state slot handed out by the scheduler;
  ``ops.group_rmsnorm`` brings the heads to unit RMS, applies the weight and the output gate.
* ``attention`` - GQA softmax attention, rotary positions on the first ``rot.dims`` elements of
  the q and k heads (``ops.rope_headnorm_cache_`` rotates and writes the K / V pages).
* ``attention_2`` - the same kernel path with per-head RMS norms of q and k, YaRN-scaled
  frequencies, values that are the un-normalised, un-rotated key projections (V pages written
  from the k columns), soft-capped scores and a sigmoid gate per head.

Feed-forwards: ``down(gelu_tanh(up h + b) ) + b`` or a mixture of SwiGLU experts routed in fp32
(``ops.moe_route_grouped``: softmax scores, a per-expert correction for the choice only, group-
limited choice, renormalised weights times a constant; identity experts return ``weight * h``)
plus a shared expert times ``sigmoid(sg . h)``.

The serving engine drives this class as it drives the other decoders (``forward`` on a step's token
rows + ``logits``); ``AttnMeta`` carries the per-step row maps (``tok_seq``, ``state_slots``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..parallel.dist import ParallelContext, get_context
from .config import GeluMlpSpec, GroupedMoeSpec, LizezenConfig, SwigluSpec
from .llama import AttnMeta


def _ceil8(n: int) -> int:
    return (n + 7) // 8 * 8


class LizezenModel:
    stateful = True                # recurrent layers keep per-sequence state in scheduler slots
    uses_decode_workspace = False
    supports_step_graphs = False   # prefill / mixed steps run eagerly (decode steps are graphs)
    supports_prefix_cache = False  # a cached page carries no recurrent state

    def __init__(self, cfg: LizezenConfig, device="cuda", dtype=torch.bfloat16,
                 pctx: Optional[ParallelContext] = None, seed: int = 0,
                 weights: Optional[Dict[str, torch.Tensor]] = None, fp8: bool = False):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lizezen runs in bfloat16 or float32")
        if fp8:
            raise NotImplementedError("FP8 projections cover the Llama-layout decoders")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.p = pctx or get_context()
        if self.p.tp_size > 1 or self.p.pp_size > 1:
            raise NotImplementedError("Lizezen runs on one GPU per replica (no TP / PP split)")
        self.fp8 = False
        self.kv_dtype, self.kv_scales = "auto", (1.0, 1.0)
        self.sequence_parallel, self.sp_min_tokens, self.split_mixed, self.moe_ws = False, 0, False, None
        att = [b.mixer for b in cfg.blocks if b.type != "mlstm"]
        self.hq, self.hkv, self.D = (att[0].heads, att[0].kv_heads, att[0].dim) if att else (1, 1, 1)
        self.n_experts = cfg.num_experts
        self.vocab_local = cfg.vocab_size
        self.runs = cfg.runs               # (layer, first of a pass) in running order
        self.k_cache: List[Optional[torch.Tensor]] = []   # per run
        self.v_cache: List[Optional[torch.Tensor]] = []
        self.rec_state: List[Optional[torch.Tensor]] = []
        self.skinny = (self.device.type == "cuda" and dtype == torch.bfloat16 and ops.skinny.enabled())
        self.mfma = True   # MFMA attention / expert kernels where they apply (bf16, tile sizes)
        if weights is None:
            weights = random_weights(cfg, seed, dtype)
        self._load(weights)

    # ------------------------------------------------------------------ weights
    def _load(self, w: Dict[str, torch.Tensor]):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        W = cfg.hidden

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
            M = torch.cat(mats)
            pad = _ceil8(M.shape[0]) - M.shape[0]
            if pad:
                M = torch.cat([M, torch.zeros(pad, M.shape[1], dtype=M.dtype, device=M.device)])
            return M.contiguous()

        def dyt(name):
            a = w[name + ".alpha"]
            if a.numel() != 1:
                raise ValueError(f"{name}.alpha: one number")
            return (float(a.float().reshape(())), vec(name, W), vec(name + ".b", W))

        def swiglu(p, s: SwigluSpec, extra=()):
            return (fused(mat(p + "gate", (s.ff, W)), mat(p + "up", (s.ff, W)), *extra), mat(p + "down", (W, s.ff)))

        self.embed = mat("embed", (cfg.vocab_size, W))
        self.w_loop = mat("loop.in", (W, 2 * W)) if cfg.loop is not None else None
        self.layers: List[dict] = []
        for i, b in enumerate(cfg.blocks):
            p, m = f"l{i}.", b.mixer
            L = {"type": b.type, "spec": m, "mlp": b.mlp, "norm": dyt(p + "norm1")}
            if b.type == "mlstm":
                nq, nv, Hh = m.heads * m.dim, m.heads * m.vdim, m.heads
                L["w_in"] = fused(mat(p + "mix.q", (nq, W)), mat(p + "mix.k", (nq, W)), mat(p + "mix.v", (nv, W)),
                                  mat(p + "mix.g", (nv, W)), mat(p + "mix.i", (Hh, W)), mat(p + "mix.f", (Hh, W)))
                L["offs"] = (0, nq, 2 * nq, 2 * nq + 2 * nv)    # q, k, v, gates; the output gate sits at 2 nq + nv
                L["gate_bias"] = torch.cat([vec(p + "mix.i.b", Hh), vec(p + "mix.f.b", Hh)])
                L["on"] = vec(p + "mix.norm", nv)
                L["wo"] = mat(p + "mix.o", (W, nv))
            elif b.type in ("attention", "attention_2"):
                nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
                parts = [mat(p + "mix.q", (nq, W)), mat(p + "mix.k", (nk, W))]
                if not m.values_from_keys:
                    parts.append(mat(p + "mix.v", (nv, W)))
                if m.head_gate:
                    L["g_off"] = sum(t.shape[0] for t in parts)
                    parts.append(mat(p + "mix.g", (m.heads, W)))
                L["w_in"] = fused(*parts)
                if m.qk_norm:
                    L["qn"], L["kn"] = vec(p + "mix.q.norm", m.dim), vec(p + "mix.k.norm", m.dim)
                freq, mag = ops.rotary_frequencies(m.rot.dims, m.rot.base, m.rot.yarn)
                L["freq"], L["mag"] = freq.to(dev), mag
                L["wo"] = mat(p + "mix.o", (W, m.heads * m.vdim))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {b.type!r}")
            f = b.mlp
            if isinstance(f, GroupedMoeSpec):
                L["router"] = mat(p + "mlp.router", (f.routed, W), torch.float32)
                L["correction"] = vec(p + "mlp.correction", f.routed)
                ex = [swiglu(f"{p}mlp.e{e}.", f.expert) for e in range(f.experts)]
                L["w13"] = torch.stack([g[:2 * f.expert.ff] for g, _ in ex]).contiguous()
                L["w2"] = torch.stack([d for _, d in ex]).contiguous()
                if f.shared is not None:
                    L["wsgu"], L["wsd"] = swiglu(p + "mlp.shared.", f.shared, (mat(p + "mlp.shared.sg", (1, W)),))
            elif isinstance(f, GeluMlpSpec):
                L["wu"], L["bu"] = mat(p + "mlp.up", (f.ff, W)), vec(p + "mlp.up.b", f.ff)
                L["wd"], L["bd"] = mat(p + "mlp.down", (W, f.ff)), vec(p + "mlp.down.b", W)
            self.layers.append(L)
        self.final_norm = dyt("final.norm")
        self.lm_head = mat("head", (cfg.vocab_size, W))

    def state_dict(self) -> Dict[str, torch.Tensor]:
        dt = self.dtype

        def dyt(out, name, n):
            out[name], out[name + ".b"] = n[1].to(dt), n[2].to(dt)
            out[name + ".alpha"] = torch.tensor(n[0], dtype=dt)

        out = {"embed": self.embed, "head": self.lm_head}
        if self.w_loop is not None:
            out["loop.in"] = self.w_loop
        dyt(out, "final.norm", self.final_norm)
        for i, L in enumerate(self.layers):
            p, m, f = f"l{i}.", L["spec"], L["mlp"]
            dyt(out, p + "norm1", L["norm"])
            Wi = L["w_in"]
            out[p + "mix.o"] = L["wo"]
            if L["type"] == "mlstm":
                nq, nv, Hh = m.heads * m.dim, m.heads * m.vdim, m.heads
                o = 2 * nq + 2 * nv
                out.update({p + "mix.q": Wi[:nq], p + "mix.k": Wi[nq:2 * nq], p + "mix.v": Wi[2 * nq:2 * nq + nv],
                            p + "mix.g": Wi[2 * nq + nv:o], p + "mix.i": Wi[o:o + Hh], p + "mix.f": Wi[o + Hh:o + 2 * Hh],
                            p + "mix.i.b": L["gate_bias"][:Hh].to(dt), p + "mix.f.b": L["gate_bias"][Hh:].to(dt),
                            p + "mix.norm": L["on"].to(dt)})
            else:
                nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
                out.update({p + "mix.q": Wi[:nq], p + "mix.k": Wi[nq:nq + nk]})
                if not m.values_from_keys:
                    out[p + "mix.v"] = Wi[nq + nk:nq + nk + nv]
                if m.head_gate:
                    out[p + "mix.g"] = Wi[L["g_off"]:L["g_off"] + m.heads]
                if m.qk_norm:
                    out.update({p + "mix.q.norm": L["qn"].to(dt), p + "mix.k.norm": L["kn"].to(dt)})
            if isinstance(f, GroupedMoeSpec):
                F = f.expert.ff
                out.update({p + "mlp.router": L["router"].to(dt), p + "mlp.correction": L["correction"].to(dt)})
                for e in range(f.experts):
                    out.update({f"{p}mlp.e{e}.gate": L["w13"][e, :F], f"{p}mlp.e{e}.up": L["w13"][e, F:],
                                f"{p}mlp.e{e}.down": L["w2"][e]})
                if f.shared is not None:
                    Fs = f.shared.ff
                    out.update({p + "mlp.shared.gate": L["wsgu"][:Fs], p + "mlp.shared.up": L["wsgu"][Fs:2 * Fs],
                                p + "mlp.shared.sg": L["wsgu"][2 * Fs:2 * Fs + 1], p + "mlp.shared.down": L["wsd"]})
            elif f is not None:
                out.update({p + "mlp.up": L["wu"], p + "mlp.up.b": L["bu"].to(dt), p + "mlp.down": L["wd"],
                            p + "mlp.down.b": L["bd"].to(dt)})
        return out

    # ------------------------------------------------------------------ cache and state
    def allocate_kv_cache(self, num_blocks: int, block_size: int = 64, kv_dtype: str = "auto",
                          kv_scales=(1.0, 1.0)):
        """Row-major pages in the model dtype, one K [blocks, kv_heads, 64, dim] and one V [blocks,
        kv_heads, 64, vdim] tensor per *run* of an attention layer (a layer of the repeated span
        has one pair per pass), all addressed by the same page numbers; ``mlstm`` runs have none."""
        if block_size != 64:
            raise ValueError("the gfx950 attention kernels use 64-token KV pages")
        if kv_dtype not in ("auto", "bf16"):
            raise ValueError("Lizezen keeps its KV pages in the model dtype")
        self.k_cache, self.v_cache = [], []
        for li, _ in self.runs:
            L = self.layers[li]
            m = L["spec"]
            if L["type"] == "mlstm":
                self.k_cache.append(None)
                self.v_cache.append(None)
            else:
                self.k_cache.append(torch.zeros(num_blocks, m.kv_heads, block_size, m.dim, device=self.device, dtype=self.dtype))
                self.v_cache.append(torch.zeros(num_blocks, m.kv_heads, block_size, m.vdim, device=self.device, dtype=self.dtype))
        return self.k_cache, self.v_cache

    def allocate_state(self, slots: int) -> None:
        """Recurrent state: per run of an ``mlstm`` layer fp32 [slots, heads, ops.mlstm_state_size]
        (S, n, m of every head). A slot needs no clearing when it is given to a new sequence: a
        segment that starts at position 0 starts from zeros, not from the slot."""
        self.rec_state = []
        for li, _ in self.runs:
            L = self.layers[li]
            m = L["spec"]
            self.rec_state.append(torch.zeros(max(1, slots), m.heads, ops.mlstm_state_size(m.dim, m.vdim),
                                              device=self.device, dtype=torch.float32) if L["type"] == "mlstm" else None)

    def kv_block_bytes(self, block_size: int = 64, kv_dtype: str = "auto") -> int:
        elem = torch.finfo(self.dtype).bits // 8
        n = 0
        for li, _ in self.runs:
            b = self.cfg.blocks[li]
            if b.type != "mlstm":
                n += b.mixer.kv_heads * (b.mixer.dim + b.mixer.vdim)
        return max(1, n) * block_size * elem

    def copy_kv_blocks(self, src, dst) -> None:
        raise NotImplementedError("beam search forks need a copy of the recurrent state")

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

    def _attend(self, q, gate, kc, vc, pos, meta: AttnMeta, H, G, dk, dv, **kw):
        """Softmax attention of a step's rows: prompt portions on the MFMA tile kernel and
        single-token rows on the page-parallel kernel where they apply (bf16, tile-sized
        heads), everything else on the row kernel."""
        if self.mfma and ops.softmax_attention_mfma_ok(q, dk, dv, H // G, 1):
            nd = meta.n_decode if meta.kind == "mixed" else (q.shape[0] if meta.kind == "decode" else 0)
            out = torch.empty(q.shape[0], H * dv, dtype=q.dtype, device=q.device)
            if nd:
                ops.softmax_attention_rows(q[:nd], kc, vc, meta.block_tables, meta.tok_seq[:nd], pos[:nd], H, G, dk,
                                           dv, max_ctx=meta.max_ctx, gate=None if gate is None else gate[:nd],
                                           out=out[:nd], **kw)
            if nd < q.shape[0]:
                ops.softmax_attention_prefill(q[nd:], kc, vc, meta.block_tables[nd:],
                                              meta.cu_q_prefill if nd else meta.cu_q, meta.ctx_lens[nd:],
                                              meta.max_q_len, H, G, dk, dv,
                                              gate=None if gate is None else gate[nd:], out=out[nd:], **kw)
            return out
        return ops.softmax_attention(q, kc, vc, meta.block_tables, meta.tok_seq, pos, H, G, dk, dv, gate=gate, **kw)

    def _mix_attention(self, ri: int, L: dict, h, pos, meta: AttnMeta):
        m = L["spec"]
        H, G, dk, dv = m.heads, m.kv_heads, m.dim, m.vdim
        proj = self._lin(h, L["w_in"])
        kc, vc = self.k_cache[ri], self.v_cache[ri]
        ops.rope_headnorm_cache_(proj, pos, meta.slots, kc, vc, H, G, dk, dv, L["freq"], L["mag"], m.rot.dims,
                                 self.cfg.eps, q_w=L.get("qn"), k_w=L.get("kn"),
                                 v_off=None if m.values_from_keys else (H + G) * dk)
        gate = proj[:, L["g_off"]:L["g_off"] + H] if m.head_gate else None
        a = self._attend(proj[:, :H * dk], gate, kc, vc, pos, meta, H, G, dk, dv, scale=m.scale, window=0,
                         softcap=m.softcap)
        return self._lin(a, L["wo"])

    def _mix_mlstm(self, ri: int, L: dict, h, pos, meta: AttnMeta):
        m = L["spec"]
        proj = self._lin(h, L["w_in"])
        o = ops.mlstm_scan(proj, L["gate_bias"], self.rec_state[ri], m.heads, m.dim, m.vdim, m.gate_cap,
                           None if meta.kind == "decode" else meta.cu_q, meta.state_slots, pos, L["offs"])
        nv = m.heads * m.vdim
        g0 = L["offs"][2] + nv
        return self._lin(ops.group_rmsnorm(o, L["on"], m.heads, self.cfg.eps, self.dtype, gate=proj[:, g0:g0 + nv]),
                         L["wo"])

    def _swiglu(self, h, wgu, wd, s: SwigluSpec, gate_col: int = -1):
        return self._lin(ops.clamped_glu(self._lin(h, wgu), s.ff, math.inf, 1.0, gate_col, shift=0.0), wd)

    def _ff(self, L: dict, h):
        """(feed-forward output rows, fp32 bias row still to be added or None)."""
        f = L["mlp"]
        if isinstance(f, GeluMlpSpec):
            return self._lin(ops.bias_gelu_tanh_(self._lin(h, L["wu"]), L["bu"]), L["wd"]), L["bd"]
        logits = ops.linear(h if h.dtype == torch.float32 else h.float(), L["router"])
        ids, wts = ops.moe_route_grouped(logits, L["correction"], f.top, f.groups, f.keep, f.scale, ws=self.moe_ws)
        shared = None
        if f.shared is not None:
            shared = self._swiglu(h, L["wsgu"], L["wsd"], f.shared, gate_col=2 * f.shared.ff)
        return ops.moe_glu_experts(h, ids, wts, L["w13"], L["w2"], math.inf, 1.0, weight_input=False, add=shared,
                                   ws=self.moe_ws, shift=0.0, identity=f.identity > 0), None

    def forward(self, ids: torch.Tensor, pos: torch.Tensor, meta: AttnMeta,
                sample_idx: Optional[torch.Tensor] = None, embed_override=None,
                layer_tap: Optional[list] = None) -> torch.Tensor:
        """Final-normed rows selected by ``sample_idx`` (all rows if None) of a step's token rows.
        ``layer_tap``: a list that receives a copy of the residual stream after every layer run."""
        if embed_override is not None:
            raise NotImplementedError("Lizezen takes token ids only")
        if meta.tok_seq is None or meta.state_slots is None:
            raise ValueError("Lizezen steps need the engine's row maps (tok_seq, state slots)")
        dt = self.dtype
        x0 = ops.embed_rows(ids, self.embed, 1.0)
        x = x0.clone() if self.w_loop is not None else x0
        h = None
        n = len(self.runs)
        for ri, (li, inject) in enumerate(self.runs):
            L = self.layers[li]
            if inject:
                h = ops.residual_dyt_(x, self._lin(ops.pack_pair(x, x0, dt), self.w_loop), None, None, L["norm"], dt,
                                      assign=True)
            elif h is None:
                h = ops.dyt_norm(x, *L["norm"], dtype=dt)
            y = (self._mix_mlstm if L["type"] == "mlstm" else self._mix_attention)(ri, L, h, pos, meta)
            y2, bias = self._ff(L, h) if L["mlp"] is not None else (None, None)
            nxt = None
            if ri + 1 < n and not self.runs[ri + 1][1]:
                nxt = self.layers[self.runs[ri + 1][0]]["norm"]
            h = ops.residual_dyt_(x, y, y2, bias, nxt, dt)
            if layer_tap is not None:
                layer_tap.append(x.clone())
        return ops.dyt_norm(x, *self.final_norm, rows=sample_idx, dtype=dt)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return ops.linear(h, self.lm_head).float()


def random_weights(cfg: LizezenConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random weights under the checkpoint's tensor names (benchmarks, tests, smoke runs)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    def around1(n):
        return (1.0 + 0.1 * torch.randn(n, generator=g)).to(dtype)

    def dyt(name):
        return {name: around1(W), name + ".b": rnd(W, std=0.05),
                name + ".alpha": (0.4 + 0.4 * torch.rand((), generator=g)).to(dtype)}

    def swiglu(p, s: SwigluSpec):
        return {p + "gate": rnd(s.ff, W, std=sd), p + "up": rnd(s.ff, W, std=sd), p + "down": rnd(W, s.ff, std=s.ff ** -0.5)}

    sd = W ** -0.5
    w = {"embed": rnd(cfg.vocab_size, W, std=1.0), "head": rnd(cfg.vocab_size, W, std=sd)}
    w.update(dyt("final.norm"))
    if cfg.loop is not None:
        w["loop.in"] = rnd(W, 2 * W, std=sd)
    for i, b in enumerate(cfg.blocks):
        p, m = f"l{i}.", b.mixer
        w.update(dyt(p + "norm1"))
        if b.type == "mlstm":
            nq, nv, Hh = m.heads * m.dim, m.heads * m.vdim, m.heads
            w.update({p + "mix.q": rnd(nq, W, std=sd), p + "mix.k": rnd(nq, W, std=sd), p + "mix.v": rnd(nv, W, std=sd),
                      p + "mix.g": rnd(nv, W, std=sd), p + "mix.i": rnd(Hh, W, std=sd), p + "mix.f": rnd(Hh, W, std=sd),
                      p + "mix.i.b": rnd(Hh, std=1.0), p + "mix.f.b": (2.0 + torch.randn(Hh, generator=g)).to(dtype),
                      p + "mix.norm": around1(nv), p + "mix.o": rnd(W, nv, std=nv ** -0.5)})
        else:
            nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            w.update({p + "mix.q": rnd(nq, W, std=sd), p + "mix.k": rnd(nk, W, std=sd),
                      p + "mix.o": rnd(W, m.heads * m.vdim, std=(m.heads * m.vdim) ** -0.5)})
            if not m.values_from_keys:
                w[p + "mix.v"] = rnd(nv, W, std=sd)
            if m.head_gate:
                w[p + "mix.g"] = rnd(m.heads, W, std=sd)
            if m.qk_norm:
                w.update({p + "mix.q.norm": around1(m.dim), p + "mix.k.norm": around1(m.dim)})
        f = b.mlp
        if isinstance(f, GroupedMoeSpec):
            w[p + "mlp.router"] = rnd(f.routed, W, std=sd)
            w[p + "mlp.correction"] = rnd(f.routed, std=0.5 / f.routed)
            for e in range(f.experts):
                w.update(swiglu(f"{p}mlp.e{e}.", f.expert))
            if f.shared is not None:
                w.update(swiglu(p + "mlp.shared.", f.shared))
                w[p + "mlp.shared.sg"] = rnd(1, W, std=sd)
        elif f is not None:
            w.update({p + "mlp.up": rnd(f.ff, W, std=sd), p + "mlp.up.b": rnd(f.ff, std=0.1),
                      p + "mlp.down": rnd(W, f.ff, std=f.ff ** -0.5), p + "mlp.down.b": rnd(W, std=0.1)})
    return w
