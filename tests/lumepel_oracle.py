"""Plain float64 implementation of the Lumepel decoder, one function per mechanism, whole
sequences, no cache, no batching. It imports nothing from the package: the tests compare the
serving path against it. Keys and values are *expanded* per head here (the product path attends
in the latent space).

Notation: ``x`` [T, width] residual rows of one sequence at positions 0 .. T-1; weights are a
dict of float64 tensors under the checkpoint's tensor names; ``cfg`` is the config.json dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rmsnorm(x, w, eps):
    return rms(x, eps) * w


def rope_frequencies(rot: dict):
    """(frequency per pair [dims / 2], factor on cos and sin). Plain: base^(-2i/dims). With a
    ``scaling`` entry the low frequencies are divided by ``factor`` along a linear ramp over the
    pair index between the pairs that turn ``fast`` and ``slow`` times in ``original`` positions,
    and cos / sin are multiplied by 0.1 ln(factor) + 1."""
    n, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / n) for i in range(n // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def pair_of(turns):
        return n * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(sc["slow"]))), n - 1)
    i = torch.arange(n // 2, dtype=F64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(v, pos, rot: dict, interleaved: bool):
    """Rotary positions on the first ``rot.dims`` elements of the last axis of ``v`` [T, ..., d];
    pairs are (2i, 2i + 1) when ``interleaved`` and (i, i + dims / 2) otherwise."""
    n = int(rot["dims"])
    f, mag = rope_frequencies(rot)
    a = pos.to(F64)[:, None] * f[None, :]                    # [T, n / 2]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [n // 2]
    c, s = (torch.cos(a) * mag).view(shape), (torch.sin(a) * mag).view(shape)
    out = v.clone()
    if interleaved:
        u, w = v[..., 0:n:2], v[..., 1:n:2]
        out[..., 0:n:2] = u * c - w * s
        out[..., 1:n:2] = w * c + u * s
    else:
        u, w = v[..., : n // 2], v[..., n // 2:n]
        out[..., : n // 2] = u * c - w * s
        out[..., n // 2:n] = w * c + u * s
    return out


def causal_softmax(scores):
    """Softmax over j <= i of scores [..., T, T]."""
    T = scores.shape[-1]
    vis = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    s = scores.masked_fill(~vis, float("-inf"))
    s = s - s.max(-1, keepdim=True).values
    e = torch.exp(s)
    return e / e.sum(-1, keepdim=True)


def latent_attention(h, w, p, m, eps, query_latent: bool, interleaved: bool):
    """Attention whose keys and values are maps of one normalised latent per token, plus one
    rotated key part shared by the heads. ``query_latent``: the query goes through a normalised
    latent of its own (``dq``, ``uq``), else straight through ``q``."""
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    if query_latent:
        cq = rmsnorm(h @ w[p + "mix.dq"].T, w[p + "mix.dq.norm"], eps)
        q = cq @ w[p + "mix.uq"].T
    else:
        q = h @ w[p + "mix.q"].T
    q = q.view(T, H, d + dr)
    kv = h @ w[p + "mix.dkv"].T
    c = rmsnorm(kv[:, :r], w[p + "mix.dkv.norm"], eps)
    pos = torch.arange(T)
    k_rot = rotate(kv[:, r:r + dr], pos, m["rot"], interleaved)          # [T, dr], all heads
    q_rot = rotate(q[:, :, d:], pos, m["rot"], interleaved)              # [T, H, dr]
    k = (c @ w[p + "mix.uk"].T).view(T, H, d)
    v = (c @ w[p + "mix.uv"].T).view(T, H, dv)
    s = torch.einsum("ihd,jhd->hij", q[:, :, :d], k) + torch.einsum("ihd,jd->hij", q_rot, k_rot)
    a = causal_softmax(s * m["scale"])
    o = torch.einsum("hij,jhd->ihd", a, v).reshape(T, H * dv)
    return o @ w[p + "mix.o"].T


def clamped_glu(h, wg, wu, wd, limit):
    """down(g * sigmoid(1.702 g) * (u + 1)), g = min(gate h, limit), u = clamp(up h, +-limit)."""
    g = torch.clamp(h @ wg.T, max=limit)
    u = torch.clamp(h @ wu.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ wd.T


def route(h, w_router, top):
    """(expert ids [T, top], weights [T, top]): sigmoid scores, the largest ``top``, as they are."""
    s = torch.sigmoid(h @ w_router.T)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val


def moe_ff(h, w, p, mlp):
    """Sum over a token's experts of expert(weight * h), plus the shared expert times a sigmoid
    gate of one number per token."""
    top = int(mlp["router"]["top"])
    idx, val = route(h, w[p + "mlp.router"], top)
    y = torch.zeros(h.shape[0], w[p + "mlp.e0.down"].shape[0], dtype=F64)
    lim = float(mlp["expert"]["limit"])
    for j in range(top):                                   # the j-th choice of every token
        for e in idx[:, j].unique().tolist():
            rows = idx[:, j] == e
            q = f"{p}mlp.e{e}."
            y[rows] += clamped_glu(h[rows] * val[rows, j:j + 1], w[q + "gate"], w[q + "up"], w[q + "down"], lim)
    sh = mlp.get("shared")
    if sh:
        q = p + "mlp.shared."
        g = torch.sigmoid(h @ w[q + "sg"].T)                             # [T, 1]
        y = y + g * clamped_glu(h, w[q + "gate"], w[q + "up"], w[q + "down"], float(sh["limit"]))
    return y


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return clamped_glu(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"], float(mlp["limit"]))
    if mlp["kind"] == "moe":
        return moe_ff(h, w, p, mlp)
    raise ValueError(mlp["kind"])


def forward(cfg: dict, weights: dict, tokens, layer_tap=None):
    """fp64 logits [T, vocab] of one sequence. ``layer_tap``: a list that receives the residual
    stream after every layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rmsnorm(x, w[p + "norm1"], eps)
        if L["type"] == "latent_attention":
            x = x + latent_attention(h, w, p, L["mixer"], eps, query_latent=True, interleaved=True)
        elif L["type"] == "latent_attention_2":
            x = x + latent_attention(h, w, p, L["mixer"], eps, query_latent=False, interleaved=False)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            x = x + feed_forward(rmsnorm(x, w[p + "norm2"], eps), w, p, L["mlp"])
        if layer_tap is not None:
            layer_tap.append(x.clone())
    z = rmsnorm(x, w["final.norm"], eps) @ w["head"].T * float(cfg.get("logit_scale", 1.0))
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(z / cap) if cap > 0 else z


def greedy(cfg: dict, weights: dict, prompt, n: int):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]
