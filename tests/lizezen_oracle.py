"""Plain float64 implementation of the Lizezen design, written from its equations: one function
per mechanism, whole sequences, no cache, no batching. It imports nothing from the package and
is what the tests compare the serving path with.

``cfg`` is the config.json dict, ``w`` a dict of tensors under the checkpoint's names.
"""
import math

import torch

F64 = torch.float64
GATE_FLOOR = 1e-6      # added to the mLSTM denominator
WEIGHT_FLOOR = 1e-20   # added to the sum of the chosen experts' scores


# ----------------------------------------------------------------------------- small pieces
def dyt(x, alpha, weight, bias):
    """Dynamic tanh in place of a norm: tanh(alpha x) * weight + bias, no statistics."""
    return torch.tanh(float(alpha) * x) * weight + bias


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def lin(x, w, b=None):
    y = x @ w.to(F64).t()
    return y if b is None else y + b.to(F64)


# ----------------------------------------------------------------------------- rotary positions
def rotary_frequencies(rot):
    """(frequency per pair, factor on cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def pair_index(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_index(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate(x, rot, first_pos=0):
    """x [T, heads, d]: element i of the first ``dims`` is paired with element i + dims / 2."""
    dims = int(rot["dims"])
    half = dims // 2
    freq, mag = rotary_frequencies(rot)
    pos = torch.arange(first_pos, first_pos + x.shape[0], dtype=F64)
    ang = pos[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


# ----------------------------------------------------------------------------- attention
def causal_attention(q, k, v, scale, softcap=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; query head h reads kv head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].t()) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def mix_attention(h, m, w, p):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rotate(lin(h, w[p + "q"]).view(T, H, d), m["rot"])
    k = rotate(lin(h, w[p + "k"]).view(T, G, d), m["rot"])
    v = lin(h, w[p + "v"]).view(T, G, dv)
    return lin(causal_attention(q, k, v, float(m["scale"])).reshape(T, H * dv), w[p + "o"])


def mix_attention_2(h, m, w, p, eps):
    """Values are the key projections as they come out of W_k; q and k get a per-head RMS norm, then
    rotary positions; capped scores; a sigmoid gate per head on the output."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = lin(h, w[p + "q"]).view(T, H, d)
    k = lin(h, w[p + "k"]).view(T, G, d)
    v = k.clone()
    q = rotate(unit_rms(q, eps) * w[p + "q.norm"].to(F64), m["rot"])
    k = rotate(unit_rms(k, eps) * w[p + "k.norm"].to(F64), m["rot"])
    a = causal_attention(q, k, v, float(m["scale"]), m.get("softcap"))
    a = a * torch.sigmoid(lin(h, w[p + "g"]))[:, :, None]
    return lin(a.reshape(T, H * d), w[p + "o"])


# ----------------------------------------------------------------------------- mLSTM
def soft_clip(z, cap):
    return cap * torch.tanh(z / cap)


def mlstm_cell(q, k, v, ig, fg):
    """One head. q, k [T, d] (q already scaled), v [T, dv], ig / fg [T] log gates. Returns [T, dv]."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=F64)
    n = torch.zeros(d, dtype=F64)
    m = 0.0
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        i, f = float(ig[t]), float(fg[t])
        m_new = max(f + m, i)
        keep, take = math.exp(f + m - m_new), math.exp(i - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        den = max(abs(float(n @ q[t])), math.exp(-m)) + GATE_FLOOR
        out[t] = (S.t() @ q[t]) / den
    return out


def mix_mlstm(h, m, w, p, eps):
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = lin(h, w[p + "q"]).view(T, H, d) * d ** -0.5
    k = lin(h, w[p + "k"]).view(T, H, d)
    v = lin(h, w[p + "v"]).view(T, H, dv)
    ig = soft_clip(lin(h, w[p + "i"], w[p + "i.b"]), cap)
    fg = torch.nn.functional.logsigmoid(soft_clip(lin(h, w[p + "f"], w[p + "f.b"]), cap))
    o = torch.stack([mlstm_cell(q[:, a], k[:, a], v[:, a], ig[:, a], fg[:, a]) for a in range(H)], dim=1)
    o = unit_rms(o, eps).reshape(T, H * dv) * w[p + "norm"].to(F64)
    return lin(o * torch.sigmoid(lin(h, w[p + "g"])), w[p + "o"])


# ----------------------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p):
    return lin(gelu_tanh(lin(h, w[p + "up"], w[p + "up.b"])), w[p + "down"], w[p + "down.b"])


def swiglu(h, w, p):
    return lin(silu(lin(h, w[p + "gate"])) * lin(h, w[p + "up"]), w[p + "down"])


def route(z, correction, r):
    """z [T, n] router logits over experts + identity experts. Returns per token a list of
    (index, weight)."""
    n = z.shape[1]
    top, scale = int(r["top"]), float(r["scale"])
    s = torch.softmax(z, dim=-1)
    c = s + correction.to(F64)
    g = r.get("groups")
    chosen = []
    for t in range(z.shape[0]):
        ct = c[t].clone()
        if g:
            per = n // int(g["count"])
            best = ct.view(int(g["count"]), per).max(dim=1).values
            kept = sorted(range(int(g["count"])), key=lambda a: (-float(best[a]), a))[:int(g["keep"])]
            for a in range(int(g["count"])):
                if a not in kept:
                    ct[a * per:(a + 1) * per] = float("-inf")
        order = sorted(range(n), key=lambda e: (-float(ct[e]), e))[:top]
        tot = sum(float(s[t, e]) for e in order) + WEIGHT_FLOOR
        chosen.append([(e, float(s[t, e]) / tot * scale) for e in order])
    return chosen


def moe_ff(h, f, w, p):
    r = f["router"]
    n_id = int(r.get("identity") or 0)
    E = int(r["experts"])
    chosen = route(lin(h, w[p + "router"]), w[p + "correction"], r)
    out = torch.zeros_like(h)
    for t, picks in enumerate(chosen):
        for e, wt in picks:
            if e >= E:
                assert e < E + n_id
                out[t] += wt * h[t]
            else:
                out[t] += wt * swiglu(h[t:t + 1], w, f"{p}e{e}.")[0]
    if f.get("shared"):
        out = out + torch.sigmoid(lin(h, w[p + "shared.sg"])) * swiglu(h, w, p + "shared.")
    return out


def feed_forward(h, f, w, p):
    if f is None:
        return torch.zeros_like(h)
    return dense_ff(h, w, p) if f.get("kind", "dense") == "dense" else moe_ff(h, f, w, p)


# ----------------------------------------------------------------------------- the model
def layer_runs(cfg):
    """Order in which the layers run: (layer index, first of a pass of the repeated span)."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, w, tokens, tap=None):
    """Logits [T, vocab] of a whole sequence; ``tap`` receives the stream after every layer run."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    x0 = x.clone()
    for li, inject in layer_runs(cfg):
        if inject:
            x = lin(torch.cat([x, x0], dim=-1), w["loop.in"])
        L, p = cfg["layers"][li], f"l{li}."
        h = dyt(x, w[p + "norm1.alpha"].to(F64), w[p + "norm1"].to(F64), w[p + "norm1.b"].to(F64))
        if L["type"] == "mlstm":
            y = mix_mlstm(h, L["mixer"], w, p + "mix.", eps)
        elif L["type"] == "attention":
            y = mix_attention(h, L["mixer"], w, p + "mix.")
        elif L["type"] == "attention_2":
            y = mix_attention_2(h, L["mixer"], w, p + "mix.", eps)
        else:
            raise ValueError(L["type"])
        x = x + (y + feed_forward(h, L.get("mlp"), w, p + "mlp."))
        if tap is not None:
            tap.append(x.clone())
    h = dyt(x, w["final.norm.alpha"].to(F64), w["final.norm"].to(F64), w["final.norm.b"].to(F64))
    return lin(h, w["head"])


def greedy(cfg, w, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]
