"""Plain-PyTorch (fp32 math) reference implementations of every HIP kernel in
``nv_genai_amd/csrc/kernels``.

They serve two purposes: the numerics oracle of the kernel tests (a GPU kernel is compared
against the op below evaluated in fp32), and the CPU execution path used by the CPU-only
unit tests of the engine / chain server. Layouts and semantics match the kernels exactly:

* paged caches: K ``[num_blocks, Hkv, BS, D]``, V transposed ``[num_blocks, Hkv, D, BS]``;
* ``qkv`` is the fused projection output ``[T, (Hq + 2*Hkv) * D]``;
* sampling uses the same counter-based RNG (splitmix64 of ``seed + golden * (ctr + 1)``) and
  Gumbel-max draw, so CPU and GPU pick identical tokens for identical logits.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * r * w.float()).to(x.dtype)


def add_rmsnorm(resid: torch.Tensor, delta: torch.Tensor, w: torch.Tensor, eps: float):
    s = (resid.float() + delta.float()).to(resid.dtype)
    resid.copy_(s)
    return rmsnorm(s, w, eps)


def layernorm(x, g, b, eps, resid=None):
    xf = x.float() + (resid.float() if resid is not None else 0.0)
    y = torch.nn.functional.layer_norm(xf, (x.shape[-1],), g.float(), b.float(), eps)
    return y.to(x.dtype)


def add_layernorm(resid, delta, g, b, eps):
    """resid += delta (stored in the residual dtype); returns LayerNorm(resid) * g + b."""
    s = (resid.float() + delta.float()).to(resid.dtype)
    resid.copy_(s)
    return layernorm(s, g, b, eps)


def gelu_tanh_mul(x: torch.Tensor) -> torch.Tensor:
    """GeGLU: x = [gate | up] -> gelu_tanh(gate) * up."""
    F = x.shape[-1] // 2
    g, u = x[..., :F].float(), x[..., F:].float()
    return (torch.nn.functional.gelu(g, approximate="tanh") * u).to(x.dtype)


def silu_mul(x: torch.Tensor) -> torch.Tensor:
    F = x.shape[-1] // 2
    g, u = x[..., :F].float(), x[..., F:].float()
    return (torch.nn.functional.silu(g) * u).to(x.dtype)


def bias_gelu_(x: torch.Tensor, bias: Optional[torch.Tensor], approximate=False) -> torch.Tensor:
    """approximate: False / "none" (erf GELU), True / "tanh", or "quick" (x * sigmoid(1.702 x))."""
    xf = x.float() + (bias.float() if bias is not None else 0.0)
    if approximate == "quick":
        y = xf * torch.sigmoid(1.702 * xf)
    else:
        y = torch.nn.functional.gelu(xf, approximate="tanh" if approximate in (True, "tanh") else "none")
    x.copy_(y.to(x.dtype))
    return x


def rope_cos_sin(max_pos: int, D: int, theta: float = 500000.0,
                 scaling: Optional[dict] = None) -> torch.Tensor:
    """[max_pos, D] fp32 table: cos of the D/2 frequencies, then sin (rotate-half layout).

    ``scaling`` implements Llama-3.1 style frequency scaling when given
    (factor, low_freq_factor, high_freq_factor, original_max_position_embeddings)."""
    inv = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    if scaling:
        factor = scaling.get("factor", 8.0)
        lo = scaling.get("low_freq_factor", 1.0)
        hi = scaling.get("high_freq_factor", 4.0)
        old = scaling.get("original_max_position_embeddings", 8192)
        wavelen = 2 * math.pi / inv
        lo_wl, hi_wl = old / lo, old / hi
        smooth = (old / wavelen - lo) / (hi - lo)
        scaled = torch.where(wavelen > lo_wl, inv / factor, inv)
        mid = (wavelen <= lo_wl) & (wavelen >= hi_wl)
        scaled = torch.where(mid, (1 - smooth) * inv / factor + smooth * inv, scaled)
        inv = scaled
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos(), f.sin()], dim=-1).float()


def _to_cache(x: torch.Tensor, cache: torch.Tensor, scale: float) -> torch.Tensor:
    """Cache element type: bf16 as is; fp8 e4m3fn stores x / scale, saturated to +-448."""
    if cache.dtype == torch.float8_e4m3fn:
        return (x.float() * (1.0 / scale)).clamp(-448.0, 448.0).to(cache.dtype)
    return x.to(cache.dtype)


def rope_cache_(qkv, pos, cos_sin, slots, kc, vc, Hq, Hkv, D, kv_scales=(1.0, 1.0)):
    T = qkv.shape[0]
    x = qkv.view(T, Hq + 2 * Hkv, D)
    cs = cos_sin[pos.long()]  # [T, D]
    c, s = cs[:, : D // 2].unsqueeze(1), cs[:, D // 2:].unsqueeze(1)
    rot = x[:, : Hq + Hkv].float()
    x1, x2 = rot[..., : D // 2], rot[..., D // 2:]
    out = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1).to(qkv.dtype)
    x[:, : Hq + Hkv] = out
    if slots is not None:
        BS = kc.shape[2]
        sl = slots.long()
        ok = sl >= 0
        blk, off = sl[ok] // BS, sl[ok] % BS
        k = x[ok, Hq: Hq + Hkv]  # [n, Hkv, D]
        v = x[ok, Hq + Hkv:]
        kc[blk, :, off, :] = _to_cache(k, kc, kv_scales[0])
        vc[blk, :, :, off] = _to_cache(v, vc, kv_scales[1])
    return qkv


def _gather_kv(kc, vc, bt_row, ctx, kvh, kv_scales=(1.0, 1.0)):
    BS = kc.shape[2]
    n_pages = (ctx + BS - 1) // BS
    blocks = bt_row[:n_pages].long()
    k = kc[blocks, kvh].reshape(-1, kc.shape[3])[:ctx]  # [ctx, D]
    v = vc[blocks, kvh].permute(0, 2, 1).reshape(-1, vc.shape[2])[:ctx]
    if kc.dtype == torch.float8_e4m3fn:
        return k.float() * kv_scales[0], v.float() * kv_scales[1]
    return k.float(), v.float()


def decode_attention(q, kc, vc, block_tables, ctx_lens, Hq, Hkv, scale, D=128, window=0,
                     kv_scales=(1.0, 1.0)):
    """One query per sequence at position ctx - 1; ``window`` > 0 keeps only the last
    ``window`` keys (sliding-window attention: key j visible iff j > ctx - 1 - window)."""
    B = ctx_lens.numel()
    G = Hq // Hkv
    out = torch.zeros(B, Hq * D, dtype=q.dtype, device=q.device)
    for b in range(B):
        ctx = int(ctx_lens[b])
        if ctx == 0:
            continue
        lo = max(0, ctx - window) if window > 0 else 0
        for kvh in range(Hkv):
            k, v = _gather_kv(kc, vc, block_tables[b], ctx, kvh, kv_scales)
            k, v = k[lo:], v[lo:]
            qs = q[b, kvh * G * D:(kvh + 1) * G * D].view(G, D).float()
            p = torch.softmax(qs @ k.T * scale, dim=-1)
            out[b, kvh * G * D:(kvh + 1) * G * D] = (p @ v).reshape(-1).to(q.dtype)
    return out


def prefill_attention_paged(q, kc, vc, block_tables, cu_q, ctx_lens, Hq, Hkv, D, scale,
                            causal=True, window=0, kv_scales=(1.0, 1.0)):
    G = Hq // Hkv
    T = q.shape[0]
    out = torch.zeros(T, Hq * D, dtype=q.dtype, device=q.device)
    B = cu_q.numel() - 1
    for b in range(B):
        s0, s1 = int(cu_q[b]), int(cu_q[b + 1])
        ql, ctx = s1 - s0, int(ctx_lens[b])
        if ql == 0:
            continue
        qpos = torch.arange(ctx - ql, ctx, device=q.device)
        kpos = torch.arange(ctx, device=q.device)
        mask = kpos[None, :] <= qpos[:, None] if causal else torch.ones(ql, ctx, dtype=torch.bool, device=q.device)
        if window > 0:
            mask = mask & (kpos[None, :] > qpos[:, None] - window)
        for hq in range(Hq):
            k, v = _gather_kv(kc, vc, block_tables[b], ctx, hq // G, kv_scales)
            qs = q[s0:s1, hq * D:(hq + 1) * D].float()
            sc = (qs @ k.T) * scale
            sc = sc.masked_fill(~mask, float("-inf"))
            out[s0:s1, hq * D:(hq + 1) * D] = (torch.softmax(sc, -1) @ v).to(q.dtype)
    return out


def prefill_attention_worklist(q, kc, vc, block_tables, cu_q, ctx_lens, Hq, Hkv, scale, items, n_items,
                               out=None, causal=True, window=0, rw=128, D=128, kv_scales=(1.0, 1.0)):
    """The work-list kernel's semantics: every listed (sequence, row block) pair writes its
    RW query rows (absolute token rows cu_q[b] + RW qb ...) of every head; other rows of
    ``out`` are left as they are."""
    G = Hq // Hkv
    if out is None:
        out = torch.zeros(q.shape[0], Hq * D, dtype=q.dtype, device=q.device)
    n = int(n_items.reshape(-1)[0])
    for b, qb in items[:n].tolist():
        s0, s1 = int(cu_q[b]), int(cu_q[b + 1])
        ql, ctx = s1 - s0, int(ctx_lens[b])
        r0, r1 = qb * rw, min(ql, qb * rw + rw)
        if r0 >= r1:
            continue
        qpos = torch.arange(ctx - ql + r0, ctx - ql + r1, device=q.device)
        kpos = torch.arange(ctx, device=q.device)
        mask = kpos[None, :] <= qpos[:, None] if causal else torch.ones(r1 - r0, ctx, dtype=torch.bool,
                                                                        device=q.device)
        if window > 0:
            mask = mask & (kpos[None, :] > qpos[:, None] - window)
        for hq in range(Hq):
            k, v = _gather_kv(kc, vc, block_tables[b], ctx, hq // G, kv_scales)
            qs = q[s0 + r0:s0 + r1, hq * D:(hq + 1) * D].float()
            sc = ((qs @ k.T) * scale).masked_fill(~mask, float("-inf"))
            out[s0 + r0:s0 + r1, hq * D:(hq + 1) * D] = (torch.softmax(sc, -1) @ v).to(out.dtype)
    return out


def varlen_attention(q, k, v, cu, Hq, Hkv, D, scale, causal=False):
    G = Hq // Hkv
    T = q.shape[0]
    out = torch.zeros(T, Hq * D, dtype=q.dtype, device=q.device)
    for b in range(cu.numel() - 1):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        n = s1 - s0
        if n == 0:
            continue
        for hq in range(Hq):
            kvh = hq // G
            qs = q[s0:s1, hq * D:(hq + 1) * D].float()
            ks = k[s0:s1, kvh * D:(kvh + 1) * D].float()
            vs = v[s0:s1, kvh * D:(kvh + 1) * D].float()
            sc = (qs @ ks.T) * scale
            if causal:
                m = torch.ones(n, n, dtype=torch.bool, device=q.device).tril()
                sc = sc.masked_fill(~m, float("-inf"))
            out[s0:s1, hq * D:(hq + 1) * D] = (torch.softmax(sc, -1) @ vs).to(q.dtype)
    return out


# ----------------------------------------------------------------------------- MoE
def moe_route(logits: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Mixtral routing: softmax over all experts (fp32), top-k, renormalised over the k.
    Returns (ids int32 [T, k], weights fp32 [T, k]) in descending-probability order."""
    p = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(p, k, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    return ids.to(torch.int32), w


def moe_ffn(x, router, w13, w2, k, expert0=0, act="silu"):
    """Sparse MoE MLP of one layer on rows x [T, H] (fp32 math per expert):
    sum_j w_j * down_e(act(gate_e(x)) * up_e(x)) over the top-k experts e of each row that
    this rank holds (experts [expert0, expert0 + w13.shape[0]))."""
    logits = (x @ router.t())
    ids, wts = moe_route(logits, k)
    E, F2, _ = w13.shape
    F = F2 // 2
    out = torch.zeros(x.shape[0], w2.shape[1], dtype=torch.float32, device=x.device)
    for e in range(E):
        tok, slot = torch.where(ids == expert0 + e)
        if tok.numel() == 0:
            continue
        gu = x[tok].float() @ w13[e].float().t()
        g, u = gu[:, :F], gu[:, F:]
        h = (torch.nn.functional.silu(g) if act == "silu" else
             torch.nn.functional.gelu(g, approximate="tanh")) * u
        y = h.to(x.dtype).float() @ w2[e].float().t()
        out.index_add_(0, tok, y * wts[tok, slot].unsqueeze(1))
    return out.to(x.dtype)


# ----------------------------------------------------------------------------- sampling
_GOLD = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def hash_uniform(seed: int, ctr: np.ndarray) -> np.ndarray:
    """Same counter RNG as common.h::hash_uniform -> float32 in (0, 1]."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + _GOLD * (ctr.astype(np.uint64) + np.uint64(1))
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return ((z >> np.uint64(40)).astype(np.float32) + np.float32(1.0)) * np.float32(1.0 / 16777216.0)


def sample(logits, temperature, top_k, top_p, seeds, steps, rep_penalty=None, history=None):
    B, V = logits.shape
    x = logits.float().clone()
    toks = torch.zeros(B, dtype=torch.int32)
    lps = torch.zeros(B, dtype=torch.float32)
    for b in range(B):
        row = x[b]
        if rep_penalty is not None and history is not None and float(rep_penalty[b]) != 1.0:
            pen = float(rep_penalty[b])
            h = history[b].long()
            h = torch.unique(h[(h >= 0) & (h < V)])
            vals = row[h]
            row[h] = torch.where(vals > 0, vals / pen, vals * pen)
        t = float(temperature[b])
        k = int(top_k[b])
        p = float(top_p[b])
        greedy = not (t > 0) or k == 1
        inv_t = 1.0 if greedy else 1.0 / t
        xs = row * inv_t
        M = xs.max()
        logZ = torch.log(torch.exp(xs - M).sum())
        if greedy:
            tok = int(torch.argmax(xs))
            toks[b], lps[b] = tok, float(xs[tok] - M - logZ)
            continue
        keep = torch.ones(V, dtype=torch.bool)
        if 0 < k < V:
            kth = torch.topk(xs, k).values[-1]
            keep &= xs >= kth
        if p < 1.0:
            pm = torch.exp(xs - M) * keep
            order = torch.argsort(xs, descending=True)
            cs = torch.cumsum(pm[order], 0)
            target = p * pm.sum()
            cut = int(torch.searchsorted(cs, target.reshape(1)).item())
            cut = min(cut, V - 1)
            thr = xs[order[cut]]
            keep &= xs >= thr
        u = torch.from_numpy(hash_uniform(int(seeds[b]), np.arange(V, dtype=np.uint64) + np.uint64(int(steps[b]) * V)))
        g = -torch.log(-torch.log(u))
        sc = torch.where(keep, xs + g, torch.tensor(float("-inf")))
        tok = int(torch.argmax(sc))
        toks[b], lps[b] = tok, float(xs[tok] - M - logZ)
    return toks.to(logits.device), lps.to(logits.device)


# ----------------------------------------------------------------------------- search
def score(Q, X, row_bias=None, dot_scale=1.0):
    S = (Q.float() @ X.float().T) * dot_scale
    if row_bias is not None:
        S = S + row_bias.float()[None, :]
    return S


def topk(S: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    k = min(k, S.shape[1])
    v, i = torch.topk(S.float(), k, dim=1)
    return v, i


def ivf_search_topk(Q, X, row_bias, dot_scale, probes, list_beg, list_end, k):
    """Per query: exact top-k over the rows of its probed lists (slab rows; -inf / -1 pads)."""
    nq = Q.shape[0]
    vals = torch.full((nq, k), float("-inf"), device=X.device)
    rows = torch.full((nq, k), -1, dtype=torch.int64, device=X.device)
    beg, end = list_beg.tolist(), list_end.tolist()
    for i in range(nq):
        rr = [torch.arange(beg[p], end[p]) for p in probes[i].tolist() if end[p] > beg[p]]
        if not rr:
            continue
        r = torch.cat(rr).to(X.device)
        s = score(Q[i:i + 1], X.index_select(0, r), None if row_bias is None else row_bias.index_select(0, r),
                  dot_scale)[0]
        kk = min(k, r.numel())
        v, j = torch.topk(s, kk)
        vals[i, :kk] = v
        rows[i, :kk] = r[j]
    return vals, rows


def embedding(ids, table, vocab_lo=0, scale=1.0):
    local = ids.long() - vocab_lo
    ok = (local >= 0) & (local < table.shape[0])
    h = torch.nn.functional.embedding(local.clamp(0, table.shape[0] - 1), table)
    h = h * ok.unsqueeze(-1).to(h.dtype)
    if scale != 1.0:
        h = h * torch.tensor(scale, dtype=h.dtype)
    return h


def pool_l2norm(hidden, cu, mode: int, normalize: bool):
    B = cu.numel() - 1
    out = torch.zeros(B, hidden.shape[1], dtype=torch.float32, device=hidden.device)
    for b in range(B):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        if s1 <= s0:
            continue
        v = hidden[s0].float() if mode == 0 else hidden[s0:s1].float().mean(0)
        if normalize:
            v = v / v.norm().clamp_min(1e-12)
        out[b] = v
    return out


def row_sqnorm(X):
    return X.float().pow(2).sum(-1)


# ---------------------------------------------------------------- DSP (FM-ASR front end)
def fir_c64(x, taps, hist=None):
    """y[i] = sum_k taps[k] x[i-k] (complex x, real taps); x[<0] from ``hist`` or zeros."""
    nt = taps.numel()
    pre = hist if hist is not None else torch.zeros(nt - 1, dtype=x.dtype, device=x.device)
    xx = torch.cat([pre.to(x.dtype), x])
    w = taps.flip(0).to(torch.float64)
    re = torch.nn.functional.conv1d(xx.real.double().view(1, 1, -1), w.view(1, 1, -1)).view(-1)
    im = torch.nn.functional.conv1d(xx.imag.double().view(1, 1, -1), w.view(1, 1, -1)).view(-1)
    return torch.complex(re.float(), im.float())


def fm_demod(x, prev=None):
    if prev is not None:
        x = torch.cat([torch.tensor([prev], dtype=x.dtype, device=x.device), x])
    d = x[1:] * x[:-1].conj()
    return torch.atan2(d.imag, d.real).float()


def resample_pcm(x, h, down, pre, nout, gain):
    """Decimating FIR y[m] = gain * sum_k h[k] x[(m + pre) * down - k]; returns (float, int16)."""
    full = torch.nn.functional.conv1d(
        torch.nn.functional.pad(x.double().view(1, 1, -1), (h.numel() - 1, h.numel() - 1)),
        h.double().flip(0).view(1, 1, -1)).view(-1)
    idx = (torch.arange(nout, dtype=torch.int64) + pre) * down
    y = torch.zeros(nout, dtype=torch.float64)
    ok = idx < full.numel()
    y[ok] = full[idx[ok]]
    y = (gain * y).float()
    pcm = (y * 32768.0).clamp(-32768.0, 32767.0).to(torch.int16)
    return y, pcm


def quant_fp8_rows(x, mode: int, Mp: int):
    """fp32 reference of the row-wise FP8 quantiser (kernels/quant.hip)."""
    xf = x.float()
    if mode == 1:
        F = xf.shape[1] // 2
        g, u = xf[:, :F], xf[:, F:]
        xf = g / (1.0 + torch.exp(-g)) * u
    M, H = xf.shape
    s = xf.abs().amax(1, keepdim=True).clamp_min(1e-12) / 448.0
    y = torch.zeros(Mp, H, dtype=torch.float8_e4m3fn)
    y[:M] = (xf / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    sp = torch.ones(Mp, 1)
    sp[:M] = s
    return y, sp


# ------------------------------------------------------------------------- post-norm fp32 residual rows
def embed_pos(ids, pos, embed, ptab):
    """fp32 rows embed[id] + ptab[pos]."""
    return embed[ids.long()].float() + ptab[pos.long()].float()


def rmsnorm_residual_(x, y, w, eps, cast_out=None):
    """x (fp32, in place) += y * rsqrt(mean(y^2) + eps) * w; ``cast_out`` takes a copy of x."""
    yf = y.float()
    x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * w)
    if cast_out is not None:
        cast_out.copy_(x)
    return x


def rmsnorm_f32(x, w, eps, rows=None, dtype=torch.float32):
    xs = x if rows is None else x.index_select(0, rows)
    return (xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + eps) * w).to(dtype)


def token_shift(x, mu, src, state, dtype):
    """h[t] = x[t] + (prev - x[t]) * mu; prev = x[src] (src >= 0), zeros (-1) or state[-(src + 2)]."""
    s = src.long()
    prev = torch.zeros_like(x)
    rows = s >= 0
    prev[rows] = x[s[rows]]
    st = s <= -2
    prev[st] = state[-(s[st] + 2)]
    return (x + (prev - x) * mu).to(dtype)


def shift_save_(state, x, last_row, slot):
    ok = (slot >= 0) & (last_row >= 0)
    state[slot[ok].long()] = x[last_row[ok].long()]
    return state


def qk_norm_cache_(proj, qw, kw, eps, slots, kc, vc, Hq, Hkv, dk, dv):
    """RMS norm over the whole q and the whole k projection (q written back in place), then the
    paged write of k and v: K [blocks, Hkv, 64, dk], V^T [blocks, Hkv, dv, 64]."""
    nq, nk, nv = Hq * dk, Hkv * dk, Hkv * dv
    q, k = proj[:, :nq].float(), proj[:, nq:nq + nk].float()
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw
    k = (k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw).to(proj.dtype)
    proj[:, :nq] = q.to(proj.dtype)
    sl = slots.long()
    ok = sl >= 0
    BS = kc.shape[2]
    blk, off = sl[ok] // BS, sl[ok] % BS
    kc[blk, :, off, :] = k[ok].view(-1, Hkv, dk)
    vc[blk, :, :, off] = proj[ok, nq + nk:nq + nk + nv].reshape(-1, Hkv, dv)
    return proj


def sigmoid_attention(q, gate, kc, vc, block_tables, tok_seq, pos, Hq, Hkv, dk, dv, scale, window, keep_first,
                      r1, r2, pb):
    """Un-normalised gated sigmoid attention over paged K / V^T with a sliding window that keeps
    the first tokens; one row at a time (reference)."""
    T = q.shape[0]
    out = torch.zeros(T, Hq * dv, dtype=torch.float32, device=q.device)
    BS = kc.shape[2]
    rep = Hq // Hkv
    heads = torch.arange(Hq, device=q.device) // rep
    for t in range(T):
        i = int(pos[t])
        if i < 0:
            continue
        bt = block_tables[int(tok_seq[t])]
        j = torch.arange(i + 1, device=q.device)
        j = j[(i - j < window) | (j < keep_first)]
        blk, off = bt[j // BS].long(), j % BS
        k = kc[blk, :, off, :].float()[:, heads]           # [n, Hq, dk]
        v = vc[blk, :, :, off].float()[:, heads]           # [n, Hq, dv]
        s = torch.einsum("hd,nhd->hn", q[t].float().view(Hq, dk), k) * scale
        s = s - r1[:, None] * torch.log1p(r2[:, None] * (i - j).float()[None, :])
        w = torch.sigmoid(s + pb[:, None])
        out[t] = torch.einsum("hn,nhd->hd", w, v).reshape(-1)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(q.dtype)


# ------------------------------------------------------------------------- softmax attention with head maps,
# gated linear recurrence, per-head norms (row-major pages: K [blocks, heads, 64, dk], V [blocks, heads, 64, dv])
def embed_rows(ids, embed, scale=1.0):
    """fp32 rows embed[id] * scale."""
    return embed[ids.long()].float() * scale


def rmsnorm_residual_next_(x, y, w, eps, next_w, out):
    """x (fp32, in place) += rmsnorm(y) * w, then out = rmsnorm(x) * next_w (weights of one or H
    elements)."""
    yf = y.float()
    x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * w)
    out.copy_(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * next_w)
    return x


def relu_sq(x):
    r = torch.relu(x.float())
    return (r * r).to(x.dtype)


def softcap_(z, cap):
    return z.copy_(cap * torch.tanh(z / cap))


def query_temperature(pos, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1) per position (fp32)."""
    return 1.0 + coef * torch.log((torch.div(pos.long() + 1, every, rounding_mode="floor") + 1).float())


def headnorm_cache_(proj, slots, kc, vc, nq, nk, dk, nv, dv, eps, q_w=None, k_w=None, bias=None, pos=None,
                    temp_coef=0.0, temp_every=1):
    """Rows [q: nq heads of dk | k: nk heads of dk | v: nv heads of dv | ...]: add ``bias``, RMS-
    normalise every q head (``q_w``) and every k head (``k_w``) over its dk elements, scale q by
    the query temperature of its position, write q and k back in place, and k / v into the
    token's page slot."""
    n0, n1, n2 = nq * dk, (nq + nk) * dk, (nq + nk) * dk + nv * dv
    T = proj.shape[0]
    seg = proj[:, :n2].float()
    if bias is not None:
        seg = seg + bias
    q, k, v = seg[:, :n0].reshape(T, nq, dk), seg[:, n0:n1].reshape(T, nk, dk), seg[:, n1:n2]
    if q_w is not None and nq:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_w
    if temp_coef != 0.0 and nq:
        q = q * query_temperature(pos, temp_coef, temp_every)[:, None, None]
    if k_w is not None and nk:
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_w
    proj[:, :n0] = q.reshape(T, n0).to(proj.dtype)
    proj[:, n0:n1] = k.reshape(T, n1 - n0).to(proj.dtype)
    proj[:, n1:n2] = v.to(proj.dtype)
    sl = slots.long()
    ok = sl >= 0
    BS = kc.shape[2]
    blk, off = sl[ok] // BS, sl[ok] % BS
    if nk:
        kc[blk, :, off, :] = k[ok].to(kc.dtype)
    if nv:
        vc[blk, :, off, :] = v[ok].reshape(-1, nv, dv).to(vc.dtype)
    return proj


def softmax_attention(q, kc, vc, block_tables, tok_seq, pos, H, G, dk, dv, scale, window=0, maps=1, lam=0.0,
                      unit_eps=None, out_scale=1.0, gate=None, v_in_k=False, softcap=0.0):
    """Softmax attention of token rows over row-major pages, one row at a time. ``maps`` score
    maps per head (q head (h, m) at column (h * maps + m) * dk, k head (h // (H / G)) * maps + m,
    v head h // (H / G)), combined as a_0 - lam * a_1; optional unit RMS per head (times
    ``out_scale``) and a per-head sigmoid gate. ``v_in_k``: the values are the first dv elements
    of the key rows. ``softcap`` > 0: scores become softcap * tanh(score / softcap)."""
    T = q.shape[0]
    out = torch.zeros(T, H, dv, dtype=torch.float32, device=q.device)
    BS = kc.shape[2]
    rep = H // G
    vh = torch.arange(H, device=q.device) // rep
    qf = q.float().view(T, H, maps, dk)
    for t in range(T):
        i = int(pos[t])
        if i < 0:
            continue
        bt = block_tables[int(tok_seq[t])]
        lo = max(0, i - window + 1) if window else 0
        j = torch.arange(lo, i + 1, device=q.device)
        blk, off = bt[j // BS].long(), j % BS
        k = kc[blk, :, off, :].float().view(-1, G, maps, dk)[:, vh]     # [n, H, maps, dk]
        v = (kc[blk, :, off, :dv] if v_in_k else vc[blk, :, off, :]).float()[:, vh]   # [n, H, dv]
        s = torch.einsum("hmd,nhmd->hmn", qf[t], k) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        a = torch.einsum("hmn,nhd->hmd", torch.softmax(s, -1), v)
        out[t] = a[:, 0] - lam * a[:, 1] if maps == 2 else a[:, 0]
    if unit_eps is not None:
        out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + unit_eps) * out_scale
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.reshape(T, H * dv).to(q.dtype)


def hgrn2_scan(proj, f_bias, lower, state, H, d, dv, cu, slots, pos):
    """Rows [q (H*d) | f (H*d) | v (H*dv)] of pre-activations -> fp32 [T, H*dv]:
    q = silu(q), f = lower + (1 - lower) * sigmoid(f + f_bias); per segment (rows cu[b] ..
    cu[b + 1], or one row each when ``cu`` is None) S <- f S + (1 - f) v^T from the state slot
    (zeros when the segment starts at position 0), o = S^T q; the slot takes the last S."""
    T = proj.shape[0]
    n = slots.numel()
    qd = H * d
    pf = proj.float()
    q = torch.nn.functional.silu(pf[:, :qd]).view(T, H, d)
    f = (lower + (1.0 - lower) * torch.sigmoid(pf[:, qd:2 * qd] + f_bias)).view(T, H, d)
    v = pf[:, 2 * qd:2 * qd + H * dv].reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=torch.float32, device=proj.device)
    for b in range(n):
        t0, t1 = (b, b + 1) if cu is None else (int(cu[b]), int(cu[b + 1]))
        if t1 <= t0:
            continue
        sl = int(slots[b])
        if int(pos[t0]) == 0 or sl < 0:
            S = torch.zeros(H, d, dv, dtype=torch.float32, device=proj.device)
        else:
            S = state[sl].clone()
        for t in range(t0, t1):
            S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        if sl >= 0:
            state[sl] = S
    return out.reshape(T, H * dv)


def group_rmsnorm(x, w, groups, eps, dtype, gate=None):
    """RMS norm of every one of ``groups`` equal column groups of fp32 rows, weight per element
    of a group (or per column of the row), written in ``dtype``; ``gate`` [T, columns]: times
    sigmoid(gate)."""
    T = x.shape[0]
    xg = x.view(T, groups, -1)
    y = xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps) * w.view(-1, xg.shape[2])
    y = y.reshape(T, -1)
    if gate is not None:
        y = y * torch.sigmoid(gate.float())
    return y.to(dtype)


# ------------------------------------------------------------------------- pre-norm fp32 stream, rotated latent
# attention, clamped GLU, sigmoid-routed experts
def residual_add_rmsnorm_(x, y, w, eps, out):
    """x (fp32, in place) += y, then out = rmsnorm(x) * w (``w`` None: the sum only)."""
    x.add_(y.float())
    if w is not None:
        out.copy_(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w)
    return x


def rotary_cos_sin(pos, freq, mag):
    """(cos, sin) [T, pairs] fp32 of angles pos * freq taken in float64, times ``mag``."""
    a = pos.to(torch.float64)[:, None] * freq.to(torch.float64)[None, :]
    return (torch.cos(a) * mag).float(), (torch.sin(a) * mag).float()


def _rotate(v, cos, sin, n, interleaved):
    """Rotary pairs on the first n elements of the last axis of fp32 ``v`` [T, ..., d]."""
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [n // 2]
    c, s = cos.view(shape), sin.view(shape)
    out = v.clone()
    if interleaved:
        a, b = v[..., 0:n:2], v[..., 1:n:2]
        out[..., 0:n:2] = a * c - b * s
        out[..., 1:n:2] = b * c + a * s
    else:
        a, b = v[..., : n // 2], v[..., n // 2:n]
        out[..., : n // 2] = a * c - b * s
        out[..., n // 2:n] = b * c + a * s
    return out


def latent_rope_cache_(proj, pos, slots, page, freq, mag, interleaved, rot_dims, rot_dim, eps, kv=None, q=None,
                       q_out=None, norm=None):
    """See :func:`nv_genai_amd.ops.latent_rope_cache_`."""
    T = proj.shape[0]
    cos, sin = rotary_cos_sin(pos.clamp(min=0), freq, mag)
    if norm is not None:
        off, n, w = norm
        v = proj[:, off:off + n].float()
        proj[:, off:off + n] = (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w).to(proj.dtype)
    if kv is not None:
        off, r, w = kv
        c = proj[:, off:off + r].float()
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w
        kr = _rotate(proj[:, off + r:off + r + rot_dim].float(), cos, sin, rot_dims, interleaved)
        sl = slots.long()
        ok = sl >= 0
        BS = page.shape[2]
        page[sl[ok] // BS, 0, sl[ok] % BS, :] = torch.cat([c, kr], 1)[ok].to(page.dtype)
    if q is not None:
        off, H, d = q
        qd = d + rot_dim
        qr = _rotate(proj[:, off:off + H * qd].float().view(T, H, qd)[:, :, d:], cos, sin, rot_dims, interleaved)
        w_out = q_out.shape[1] // H
        q_out.view(T, H, w_out)[:, :, w_out - rot_dim:] = qr.to(q_out.dtype)
    return proj


def clamped_glu(x, F, limit, alpha, gate_col=-1, shift=1.0):
    """Rows [gate F | up F | ...] -> g * sigmoid(alpha g) * (u + shift), g = min(gate, limit),
    u = clamp(up, +-limit); times sigmoid(x[:, gate_col]) when gate_col >= 0."""
    xf = x.float()
    g = xf[:, :F].clamp(max=limit)
    u = xf[:, F:2 * F].clamp(min=-limit, max=limit)
    y = g * torch.sigmoid(alpha * g) * (u + shift)
    if gate_col >= 0:
        y = y * torch.sigmoid(xf[:, gate_col:gate_col + 1])
    return y.to(x.dtype)


def moe_route_scores(logits, k, score="sigmoid", renorm=False):
    """(ids int32 [T, k], weights fp32 [T, k]): the k largest ``score(logits)`` per row in
    descending order (ties: the lower expert index first), renormalised over the k or as they are."""
    lf = logits.float()
    s = torch.sigmoid(lf) if score == "sigmoid" else torch.softmax(lf, -1)
    # the activation is monotonic: choose by the logits (exact ties cannot flip through rounding)
    _, ids = torch.sort(lf, dim=-1, descending=True, stable=True)
    ids = ids[:, :k]
    w = torch.gather(s, 1, ids)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return ids.to(torch.int32), w


def moe_glu_experts(x, ids, wts, w13, w2, limit, alpha, weight_input=True, add=None, shift=1.0, identity=False):
    """Sum over a row's experts e of expert_e(x) with the routing weight on the expert's input
    (``weight_input``) or on its output; expert = clamped GLU, ``w13`` [E, 2F, H] = [gate | up],
    ``w2`` [E, H, F]. ``add`` [T, H] is added to the sum. ``identity``: ids >= E return the row
    itself times the weight."""
    E, F2, _ = w13.shape
    F = F2 // 2
    out = torch.zeros(x.shape[0], w2.shape[1], dtype=torch.float32, device=x.device)
    for e in range(E):
        tok, slot = torch.where(ids == e)
        if tok.numel() == 0:
            continue
        wt = wts[tok, slot].unsqueeze(1)
        gu = (x[tok].float() @ w13[e].float().t()) * (wt if weight_input else 1.0)
        h = clamped_glu(gu, F, limit, alpha, shift=shift).to(x.dtype)
        y = h.float() @ w2[e].float().t()
        out.index_add_(0, tok, y if weight_input else y * wt)
    if identity:
        out = out + x.float() * (wts * (ids >= E)).sum(-1, keepdim=True)
    if add is not None:
        out = out + add.float()
    return out.to(x.dtype)


# ------------------------------------------------------------------------- dynamic-tanh stream, rotary attention with
# head norms, mLSTM, group-limited routing
def dyt_norm(x, alpha, w, b, rows=None, dtype=torch.float32):
    """tanh(alpha x) * w + b of fp32 rows (``rows``: only these), in ``dtype``."""
    xr = x if rows is None else x.index_select(0, rows)
    return (torch.tanh(alpha * xr) * w + b).to(dtype)


def residual_dyt_(x, y1, y2, bias, norm, out, assign=False):
    """fp32 stream in place: ``x += y1 (+ y2) (+ bias)`` (the sub-layer outputs are summed first), or
    ``x = y1`` when ``assign``; ``norm`` = (alpha, w, b): ``out`` takes tanh(alpha x) * w + b."""
    if assign:
        x.copy_(y1.float())
    else:
        y = y1.float()
        if y2 is not None:
            y = y + y2.float()
        if bias is not None:
            y = y + bias
        x.add_(y)
    if norm is not None:
        out.copy_(torch.tanh(norm[0] * x) * norm[1] + norm[2])
    return x


def pack_pair(a, b, dtype):
    """[a | b] rows of two fp32 streams, in ``dtype``."""
    return torch.cat([a, b], dim=1).to(dtype)


def bias_gelu_tanh_(x, bias):
    """x = gelu_tanh(x + bias) in place (fp32 math; ``bias`` fp32 or None)."""
    xf = x.float() if bias is None else x.float() + bias
    x.copy_(torch.nn.functional.gelu(xf, approximate="tanh").to(x.dtype))
    return x


def rope_headnorm_cache_(proj, pos, slots, kc, vc, H, G, dk, dv, freq, mag, rot_dims, eps, q_w=None, k_w=None,
                         v_off=None):
    """See :func:`nv_genai_amd.ops.rope_headnorm_cache_`."""
    T = proj.shape[0]
    n0, n1 = H * dk, (H + G) * dk
    q = proj[:, :n0].float().view(T, H, dk)
    k = proj[:, n0:n1].float().view(T, G, dk)
    v = k.clone() if v_off is None else proj[:, v_off:v_off + G * dv].float().view(T, G, dv)
    if q_w is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_w
    if k_w is not None:
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_w
    cos, sin = rotary_cos_sin(pos.clamp(min=0), freq, mag)
    q, k = _rotate(q, cos, sin, rot_dims, False), _rotate(k, cos, sin, rot_dims, False)
    proj[:, :n0] = q.reshape(T, n0).to(proj.dtype)
    proj[:, n0:n1] = k.reshape(T, n1 - n0).to(proj.dtype)
    sl = slots.long()
    ok = sl >= 0
    BS = kc.shape[2]
    blk, off = sl[ok] // BS, sl[ok] % BS
    kc[blk, :, off, :] = k[ok].to(kc.dtype)
    vc[blk, :, off, :] = v[ok].to(vc.dtype)
    return proj


def mlstm_scan(proj, gate_bias, state, H, d, dv, cap, cu, slots, pos, offs):
    """See :func:`nv_genai_amd.ops.mlstm_scan`."""
    T = proj.shape[0]
    n = slots.numel()
    qo, ko, vo, io = offs
    pf = proj.float()
    q = pf[:, qo:qo + H * d].reshape(T, H, d) * (d ** -0.5)
    k = pf[:, ko:ko + H * d].reshape(T, H, d)
    v = pf[:, vo:vo + H * dv].reshape(T, H, dv)
    z = pf[:, io:io + 2 * H] + gate_bias
    z = cap * torch.tanh(z / cap)
    ig, fg = z[:, :H], torch.nn.functional.logsigmoid(z[:, H:])
    out = torch.zeros(T, H, dv, dtype=torch.float32, device=proj.device)
    for b in range(n):
        t0, t1 = (b, b + 1) if cu is None else (int(cu[b]), int(cu[b + 1]))
        if t1 <= t0:
            continue
        sl = int(slots[b])
        if int(pos[t0]) == 0 or sl < 0:
            S = torch.zeros(H, d, dv, dtype=torch.float32, device=proj.device)
            nn = torch.zeros(H, d, dtype=torch.float32, device=proj.device)
            m = torch.zeros(H, dtype=torch.float32, device=proj.device)
        else:
            st = state[sl]
            S, nn, m = st[:, :d * dv].reshape(H, d, dv).clone(), st[:, d * dv:d * dv + d].clone(), st[:, d * dv + d].clone()
        for t in range(t0, t1):
            m_new = torch.maximum(fg[t] + m, ig[t])
            a, bb = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
            S = a[:, None, None] * S + bb[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
            nn = a[:, None] * nn + bb[:, None] * k[t]
            m = m_new
            den = torch.maximum((nn * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
        if sl >= 0:   # S, then the copies of (n, m) the kernel's layout holds (one per 16 value columns)
            nm = torch.cat([nn, m[:, None]], dim=1)
            state[sl] = torch.cat([S.reshape(H, d * dv)] + [nm] * (-(-dv // 16)), dim=1)
    return out.reshape(T, H * dv)


def moe_route_grouped(logits, correction, k, groups, keep, scale):
    """See :func:`nv_genai_amd.ops.moe_route_grouped`."""
    T, E = logits.shape
    s = torch.softmax(logits.float(), -1)
    c = s + correction
    if groups > 1:
        per = E // groups
        best = c.view(T, groups, per).max(-1).values
        _, gi = torch.sort(best, dim=-1, descending=True, stable=True)
        kept = torch.zeros(T, groups, dtype=torch.bool, device=logits.device)
        kept.scatter_(1, gi[:, :keep], True)
        c = c.masked_fill(~kept.repeat_interleave(per, dim=1), float("-inf"))
    _, ids = torch.sort(c, dim=-1, descending=True, stable=True)
    ids = ids[:, :k]
    w = torch.gather(s, 1, ids)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * scale
    return ids.to(torch.int32), w
