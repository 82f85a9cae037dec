"""Lizezen on the serving engine against the plain oracle (tests/lizezen_oracle.py).

Every case runs on the CPU (the engine on the fp32 reference ops: scheduling, pages, state slots,
row maps) and, marked ``gpu``, on the HIP kernels in float32 and bfloat16. The models are small
random ones built here; sizes are chosen so that heads, dims, expert counts, groups and the page
size do not coincide (``odd``: a rotation on part of the head, a layer without feed-forward, a
mixture without a shared expert and without groups, a repeated span in the middle), or so that the
MFMA tile kernels run (``tiles``: the repeated span starts at the first layer).
"""
import json
import math

import pytest
import torch

import lizezen_oracle as O
from nv_genai_amd import ops
from nv_genai_amd.engine.llm_engine import EngineConfig, LLMEngine, SamplingParams
from nv_genai_amd.models.config import LizezenConfig, lizezen_layers
from nv_genai_amd.models.lizezen import LizezenModel, random_weights

GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVICES = ["cpu", GPU]
DTYPES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
          pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}


def dense(ff=24):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=3, ff=14, identity=1, groups=(3, 2), scale=1.7, shared=12):
    r = {"experts": experts, "top": top, "identity": identity, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "router": r, "expert": {"ff": ff}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def mlstm(heads=3, dim=5, vdim=7, cap=6.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def att(heads=6, kv=2, dim=10, vdim=6, dims=6, base=100.0, scale=0.3, mlp=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                                           "rot": {"base": base, "dims": dims}}, "mlp": mlp}


def att2(heads=4, kv=2, dim=12, dims=8, base=50.0, scale=0.25, cap=5.0, scaling=YARN, mlp=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(scaling)
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale, "rot": rot}
    if cap:
        m["softcap"] = cap
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def cfg_dict(layers, width=40, vocab=97, eps=1e-5, loop=None):
    d = {"architecture": "Lizezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


def cfg_odd():
    return cfg_dict([mlstm(mlp=dense()), att(mlp=moe()), att2(), mlstm(heads=2, dim=9, vdim=4, cap=11.0,
                                                                      mlp=moe(3, 2, 7, 0, None, 1.0, None)),
                     att2(heads=3, kv=3, dim=6, dims=6, scaling=None, cap=0.0, mlp=dense(9))], loop=(1, 4, 2))


def cfg_tiles():
    """Sizes the MFMA kernels take: 128 / 64-wide heads with GQA, a soft-capped 64-wide layer,
    experts of 128 on a width of 256; the repeated span starts at the first layer."""
    return cfg_dict([mlstm(heads=4, dim=64, vdim=64, cap=12.0, mlp=moe(4, 2, 128, 2, (2, 1), 1.5, 64)),
                     att(heads=8, kv=2, dim=128, vdim=64, dims=64, base=10000.0, scale=0.09, mlp=dense(64)),
                     att2(heads=4, kv=2, dim=64, dims=64, base=1000.0, scale=0.125, cap=10.0,
                          scaling={"factor": 8.0, "original": 64, "fast": 16.0, "slow": 1.0}, mlp=dense(32))],
                    width=256, loop=(0, 2, 3))


CFGS = {"odd": cfg_odd, "tiles": cfg_tiles}


def build(device, dtype="float32", seed=0, pages=24, seqs=4, cd=None, graphs=None, **eng):
    cd = cd or cfg_odd()
    cfg = LizezenConfig.from_dict(cd)
    w = random_weights(cfg, seed, torch.bfloat16)       # bf16 values, as a checkpoint holds them
    for k in w:
        if k.endswith("mlp.router"):
            w[k] = w[k] * 4.0                           # wide logits: few near ties between experts
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    model = LizezenModel(cfg, device, tdt, weights=w)
    kw = dict(model="lizezen-test", dtype=dtype, max_num_seqs=seqs, max_batched_tokens=512, max_model_len=512,
              kv_cache_blocks=pages, detokenize=False, use_graphs=(device == "cuda") if graphs is None else graphs,
              graph_batch_sizes=(1, 2, 4), mixed_graphs=False, logits_tap=True, tuned_gemms=False, async_decode=False)
    kw.update(eng)
    e = LLMEngine(EngineConfig(**kw), device=device, model=model)
    return e, cd, w


def tokens(n, vocab=97, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def close(got, want, dtype, what=""):
    got, want = got.double().cpu(), want.double()
    err = (got - want).abs().max().item() / max(1.0, want.abs().max().item())
    assert err < tol(dtype), f"{what}: relative error {err:.3e}"


def close_rows(got, want, dtype, what=""):
    """Model outputs, one row per token. In bfloat16 the router reads rounded activations, so a token
    whose k-th and (k+1)-th choice nearly tie may take another expert than the oracle does: there
    the comparison allows a few rows (two, or 3 %) to differ; every other row, and every row in
    float32, must agree. (The test models' routers are scaled up so that near ties are rare.)"""
    if dtype == "float32":
        return close(got, want, dtype, what)
    got, want = got.double().cpu(), want.double()
    err = (got - want).abs().flatten(1).max(dim=1).values / max(1.0, want.abs().max().item())
    bad = int((err >= tol(dtype)).sum())
    assert bad <= max(2, 0.03 * err.numel()), f"{what}: {bad} of {err.numel()} rows differ (worst {err.max().item():.3e})"


def tdtype(dtype):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]


def replay_cuts(eng, toks, cuts, rid=1, finish=True):
    """Feed ``toks`` in portions of the given sizes (the rest one token at a time); all logits."""
    out, at, cuts = [], 0, list(cuts)
    while at < len(toks):
        n = min(cuts.pop(0) if cuts else 1, len(toks) - at)
        done = at + n == len(toks)
        out.append(eng.replay_step([(rid, toks[at:at + n], list(range(n)))], [rid] if done and finish else []))
        at += n
    return torch.cat(out)


# ---------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_dynamic_tanh_stream_ops(device, dtype):
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(3)
    T, H = 37, 41
    x0 = 3.0 * torch.randn(T, H, generator=g)
    y1, y2 = torch.randn(T, H, generator=g).to(tdt), torch.randn(T, H, generator=g).to(tdt)
    bias, w, b = torch.randn(H, generator=g), 1.0 + 0.2 * torch.randn(H, generator=g), 0.3 * torch.randn(H, generator=g)
    alpha = 0.37
    dv = lambda t: t.to(device)   # noqa: E731
    x = dv(x0.clone())
    h = ops.residual_dyt_(x, dv(y1), dv(y2), dv(bias), (alpha, dv(w), dv(b)), tdt)
    xs = x0.double() + (y1.double() + y2.double() + bias.double())
    close(x, xs, "float32", "the sum stays fp32")
    close(h, O.dyt(xs, alpha, w.double(), b.double()), dtype, "dynamic tanh of the sum")
    assert ops.residual_dyt_(x, dv(y1), None, None, None, tdt) is None
    close(x, xs + y1.double(), "float32", "one source, no norm")
    h = ops.residual_dyt_(x, dv(y2), None, None, (alpha, dv(w), dv(b)), tdt, assign=True)
    close(x, y2.double(), "float32", "a projection replaces the stream")
    close(h, O.dyt(y2.double(), alpha, w.double(), b.double()), dtype, "norm of the replaced stream")
    rows = torch.tensor([5, 0, 36, 5])
    close(ops.dyt_norm(dv(x0), alpha, dv(w), dv(b), rows=dv(rows), dtype=tdt),
          O.dyt(x0.double()[rows], alpha, w.double(), b.double()), dtype, "gathered rows")
    close(ops.dyt_norm(dv(x0), alpha, dv(w), dv(b), dtype=tdt), O.dyt(x0.double(), alpha, w.double(), b.double()), dtype,
          "all rows")
    a, c = torch.randn(T, H, generator=g), torch.randn(T, 13, generator=g)
    close(ops.pack_pair(dv(a), dv(c), tdt), torch.cat([a, c], 1).to(tdt), "float32", "packed pair")
    for F in (23, 24):     # the scalar form and the 8-wide form
        z = (2.0 * torch.randn(T, F, generator=g)).to(tdt)
        bz = torch.randn(F, generator=g)
        close(ops.bias_gelu_tanh_(dv(z.clone()), dv(bz)), O.gelu_tanh(z.double() + bz.double()), dtype, f"gelu {F}")
        close(ops.bias_gelu_tanh_(dv(z.clone()), None), O.gelu_tanh(z.double()), dtype, f"gelu without bias {F}")
    # head norm with a weight per column and a gate; SwiGLU as the unclamped, unshifted GLU
    o = torch.randn(T, 3 * 7, generator=g)
    wn, gate = 1 + 0.1 * torch.randn(21, generator=g), torch.randn(T, 30, generator=g).to(tdt)
    want = (O.unit_rms(o.double().view(T, 3, 7), 1e-5).reshape(T, 21) * wn.double()
            * torch.sigmoid(gate[:, 4:25].double()))
    close(ops.group_rmsnorm(dv(o), dv(wn), 3, 1e-5, tdt, gate=dv(gate)[:, 4:25]), want, dtype, "gated head norm")
    for F, pad in ((23, 3), (24, 8)):
        gu = (2.0 * torch.randn(T, 2 * F + pad, generator=g)).to(tdt)
        want = O.silu(gu[:, :F].double()) * gu[:, F:2 * F].double()
        close(ops.clamped_glu(dv(gu), F, math.inf, 1.0, shift=0.0), want, dtype, "swiglu")
        close(ops.clamped_glu(dv(gu), F, math.inf, 1.0, gate_col=2 * F + 1, shift=0.0),
              want * torch.sigmoid(gu[:, 2 * F + 1:2 * F + 2].double()), dtype, "swiglu with a row gate")


def test_rotary_frequencies_against_the_oracle():
    for rot in ({"dims": 8, "base": 50.0}, {"dims": 4, "base": 100.0, "scaling": YARN},
                {"dims": 96, "base": 1e6, "scaling": {"factor": 16.0, "original": 1024, "fast": 32.0, "slow": 1.0}}):
        sc = rot.get("scaling")
        f, mag = ops.rotary_frequencies(rot["dims"], rot["base"],
                                        None if not sc else (sc["factor"], sc["original"], sc["fast"], sc["slow"]))
        fo, mo = O.rotary_frequencies(rot)
        assert torch.allclose(f, fo, rtol=1e-14, atol=0) and abs(mag - mo) < 1e-15


@pytest.mark.parametrize("sizes", [(4, 2, 10, 6, 7, 3), (5, 2, 32, 32, 16, 8), (3, 3, 128, 128, 64, 0), (9, 1, 16, 16, 8, 8)])
@pytest.mark.parametrize("from_keys", [False, True])
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_head_norm_rotation_and_page_write(device, dtype, from_keys, sizes):
    """Positions far out (the angle must stay exact), a rotation on part of the head or on all of
    it (sizes the 16-byte form takes, more heads than one round of a wave holds), slots in several
    pages, a row that is not written; values from their own columns or from the keys as projected
    (before norm and rotation)."""
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(5)
    H, G, dk, dims, dv, pad = sizes
    T = 9
    dv = dk if from_keys else dv
    rot = {"dims": dims, "base": 30.0, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}
    freq, mag = ops.rotary_frequencies(dims, 30.0, (4.0, 16, 4.0, 1.0))
    cols = (H + G) * dk + (0 if from_keys else G * dv) + pad
    proj0 = torch.randn(T, cols, generator=g).to(tdt)
    pos = torch.tensor([0, 1, 63, 64, 1000, 65535, 99999, 7, 2], dtype=torch.int32)
    slots = torch.tensor([0, 1, 63, 64, 130, 191, 5, -1, 70], dtype=torch.int32)
    qw, kw = (None, None) if not from_keys else (1 + 0.1 * torch.randn(dk, generator=g), 1 + 0.1 * torch.randn(dk, generator=g))
    kc = torch.zeros(3, G, 64, dk, dtype=tdt, device=device)
    vc = torch.zeros(3, G, 64, dv, dtype=tdt, device=device)
    proj = proj0.clone().to(device)
    ops.rope_headnorm_cache_(proj, pos.to(device), slots.to(device), kc, vc, H, G, dk, dv, freq.to(device), mag, dims, 1e-5,
                             q_w=None if qw is None else qw.to(device), k_w=None if kw is None else kw.to(device),
                             v_off=None if from_keys else (H + G) * dk)
    pd = proj0.double()
    q, k = pd[:, :H * dk].view(T, H, dk), pd[:, H * dk:(H + G) * dk].view(T, G, dk)
    v = k if from_keys else pd[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv)
    if from_keys:
        q, k = O.unit_rms(q, 1e-5) * qw.double(), O.unit_rms(k, 1e-5) * kw.double()

    def rotated(x):      # the oracle rotates whole sequences from position 0: one call per row
        return torch.stack([O.rotate(x[t:t + 1], rot, int(pos[t]))[0] for t in range(T)])

    qr, kr = rotated(q), rotated(k)
    close(proj[:, :H * dk], qr.reshape(T, -1), dtype, "rotated queries")
    close(proj[:, H * dk:(H + G) * dk], kr.reshape(T, -1), dtype, "rotated keys")
    assert torch.equal(proj[:, (H + G) * dk:].cpu(), proj0[:, (H + G) * dk:]), "the other columns stay"
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            close(kc[s // 64, :, s % 64], kr[t], dtype, f"K page row of token {t}")
            close(vc[s // 64, :, s % 64], v[t], dtype, f"V page row of token {t}")
    written = torch.zeros(192, dtype=torch.bool)
    written[slots[slots >= 0].long()] = True
    assert float(kc.transpose(1, 2).reshape(192, -1)[~written.to(kc.device)].abs().max()) == 0.0


def _pages(rows, device, tdt, bt_row, nb):
    """Token rows [n, G, d] laid into pages [nb, G, 64, d] through the block-table row."""
    n, G, d = rows.shape
    page = torch.zeros(nb, G, 64, d, dtype=tdt, device=device)
    j = torch.arange(n)
    page[bt_row[j // 64].long(), :, j % 64] = rows.to(tdt).to(device)
    return page


def o_attention(q, K, V, scale, cap, pos, gate=None):
    """Plain form: query t at position pos[t] sees rows 0 .. pos[t]; q [T, H, d], K [n, G, d], V [n, G, dv]."""
    T, H, _ = q.shape
    G = K.shape[1]
    out = torch.zeros(T, H, V.shape[2], dtype=torch.float64)
    for t in range(T):
        for h in range(H):
            kk, vv = K[: int(pos[t]) + 1, h // (H // G)].double(), V[: int(pos[t]) + 1, h // (H // G)].double()
            s = (kk @ q[t, h].double()) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            out[t, h] = torch.softmax(s, -1) @ vv
            if gate is not None:
                out[t, h] *= torch.sigmoid(gate[t, h].double())
    return out.reshape(T, -1)


@pytest.mark.parametrize("shape", [(6, 2, 10, 6, 5.0), (4, 2, 64, 64, 10.0), (8, 2, 128, 64, 0.0), (9, 3, 96, 64, 8.0),
                                   (2, 2, 128, 128, 30.0), (1, 1, 13, 13, 0.0), (4, 4, 80, 80, 12.0)])
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_one_key_stands_out_capped_scores(device, dtype, shape):
    """One key is made to match a scaled query: far back, on both sides of page borders, at the
    query's own position, and one position *after* the query (it must not be seen). With a soft cap
    the hot score saturates at the cap, so the hot key's share is what the cap leaves it - the
    comparison with the plain form shows a cap that is left out. Through the row kernel, the
    single-token kernel and the prompt kernel, with the per-head gate."""
    H, G, dk, dv, cap = shape
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(11)
    n = 700
    K = (0.3 * torch.randn(n, G, dk, generator=g)).to(tdt).float()
    V = torch.randn(n, G, dv, generator=g).to(tdt).float()
    bt = torch.randperm(16, generator=g)[:11].to(torch.int32)
    qpos = [699, 640, 128, 127, 64, 63, 5, 0]
    scale = dk ** -0.5
    for hot in (3, 63, 64, 127, 128, 576, 639, None):
        KK = K.clone()
        u = torch.randn(dk, generator=g)
        u = u / u.norm()
        if hot is not None:
            KK[hot, 0] = (6.0 * u).to(tdt).float()
        kc, vc = _pages(KK, device, tdt, bt, 16), _pages(V, device, tdt, bt, 16)
        q = 0.3 * torch.randn(len(qpos), H, dk, generator=g)
        if hot is not None:
            q[:, 0] = 40.0 * u / scale / 6.0      # head 0 (kv head 0): score 40 on the hot key
        q = q.to(tdt)
        gate = torch.randn(len(qpos), H, generator=g).to(tdt)
        pos = torch.tensor(qpos, dtype=torch.int32)
        want = o_attention(q.float(), KK, V, scale, cap, pos, gate.float())
        qd = q.reshape(len(qpos), H * dk).to(device)
        seq = torch.zeros(len(qpos), dtype=torch.int32, device=device)
        btd = bt.view(1, -1).to(device)
        kw = dict(scale=scale, softcap=cap, gate=gate.to(device))
        got = ops.softmax_attention(qd, kc, vc, btd, seq, pos.to(device), H, G, dk, dv, **kw)
        close(got, want, dtype, f"row form, hot key {hot}")
        got = ops.softmax_attention_rows(qd, kc, vc, btd, seq, pos.to(device), H, G, dk, dv, max_ctx=704, **kw)
        close(got, want, dtype, f"single-token form, hot key {hot}")
        if hot is not None and not cap:
            for t, p in enumerate(qpos):
                sg = torch.sigmoid(gate[t, 0].double())
                hit = (got[t, :dv].double().cpu() - sg * V[hot, 0].double()).abs().max().item() < 0.05
                assert hit == (hot <= p), f"query at {p}, hot key at {hot}: seen={hit}"
    # a portion: queries at positions 560 .. 699 of the same sequence in one launch
    KK = K.clone()
    u = torch.randn(dk, generator=g)
    u = u / u.norm()
    KK[600, G - 1] = (6.0 * u).to(tdt).float()
    kc, vc = _pages(KK, device, tdt, bt, 16), _pages(V, device, tdt, bt, 16)
    nq = 140
    q = 0.3 * torch.randn(nq, H, dk, generator=g)
    q[:, H - 1] = 40.0 * u / scale / 6.0
    q = q.to(tdt)
    pos = torch.arange(560, 700, dtype=torch.int32)
    want = o_attention(q.float(), KK, V, scale, cap, pos)
    cu = torch.tensor([0, nq], dtype=torch.int32, device=device)
    ctx = torch.tensor([700], dtype=torch.int32, device=device)
    got = ops.softmax_attention_prefill(q.reshape(nq, H * dk).to(device), kc, vc, bt.view(1, -1).to(device), cu, ctx, nq,
                                        H, G, dk, dv, scale=scale, softcap=cap)
    close(got, want, dtype, "portion")
    if not cap:
        for t in (39, 40, 41):     # positions 599 (the key comes one later), 600, 601
            hit = (got[t, (H - 1) * dv:].double().cpu() - V[600, G - 1].double()).abs().max().item() < 0.05
            assert hit == (t >= 40)


def o_mlstm(proj, bias, H, d, dv, cap, offs):
    """The oracle's cell on projection rows laid out as the scan op takes them."""
    T = proj.shape[0]
    qo, ko, vo, go = offs
    p = proj.double()
    ig = O.soft_clip(p[:, go:go + H] + bias[:H].double(), cap)
    fg = torch.nn.functional.logsigmoid(O.soft_clip(p[:, go + H:go + 2 * H] + bias[H:].double(), cap))
    return torch.stack([O.mlstm_cell(p[:, qo + h * d:qo + (h + 1) * d] * d ** -0.5, p[:, ko + h * d:ko + (h + 1) * d],
                                     p[:, vo + h * dv:vo + (h + 1) * dv], ig[:, h], fg[:, h]) for h in range(H)],
                       dim=1).reshape(T, H * dv)


@pytest.mark.parametrize("shape", [(3, 5, 7), (2, 9, 4), (4, 64, 64), (1, 1, 1), (2, 130, 20), (2, 32, 100)])
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_mlstm_scan_portions_and_slots(device, dtype, shape):
    """The scan in portions of many sizes and as single rows against the whole-sequence cell: the
    state (S, n, m) must come back from its slot. A stale slot is not read by a sequence that
    starts at position 0; a slot of -1 neither reads nor writes. Gate pre-activations are wide
    enough that both branches of the running maximum and the cap are taken."""
    H, d, dv = shape
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(13)
    T, cap = 83, 6.0
    nq, nv = H * d, H * dv
    offs = (2, 2 + nq, 2 + 2 * nq, 2 + 2 * nq + nv + 3)
    cols = offs[3] + 2 * H + 1
    proj = torch.randn(T, cols, generator=g)
    proj[:, offs[3]:offs[3] + 2 * H] *= 4.0
    proj = proj.to(tdt)
    bias = torch.randn(2 * H, generator=g)
    want = o_mlstm(proj.float(), bias, H, d, dv, cap, offs)
    state = torch.full((3, H, ops.mlstm_state_size(d, dv)), 7.0, device=device)     # stale
    pd, bd = proj.to(device), bias.to(device)

    def run(t0, t1, slot, single=False):
        n = t1 - t0
        pos = torch.arange(t0, t1, dtype=torch.int32, device=device)
        if single:
            return ops.mlstm_scan(pd[t0:t1], bd, state, H, d, dv, cap, None,
                                  torch.full((n,), slot, dtype=torch.int32, device=device)[:1] if n == 1 else None, pos, offs)
        cu = torch.tensor([0, n], dtype=torch.int32, device=device)
        return ops.mlstm_scan(pd[t0:t1], bd, state, H, d, dv, cap, cu, torch.tensor([slot], dtype=torch.int32, device=device),
                              pos, offs)

    cuts = [0, 1, 20, 22, 27, 43, 44, 60]
    got = [run(a, b, 1) for a, b in zip(cuts, cuts[1:])]
    got += [run(t, t + 1, 1, single=True) for t in range(60, T)]
    close(torch.cat(got), want, dtype, "portions, then single rows")
    assert float((state[0] - 7.0).abs().max()) == 0.0 and float((state[2] - 7.0).abs().max()) == 0.0
    keep = state.clone()
    out = run(0, 30, -1)
    close(out, want[:30], dtype, "no slot")
    assert torch.equal(keep, state)
    # two segments of different sequences in one launch, one continuing from its slot
    run(0, 40, 2)
    cu = torch.tensor([0, 43, 60], dtype=torch.int32, device=device)
    pos = torch.cat([torch.arange(40, 83), torch.arange(0, 17)]).to(torch.int32).to(device)
    rows = torch.cat([pd[40:83], pd[0:17]])
    out = ops.mlstm_scan(rows, bd, state, H, d, dv, cap, cu, torch.tensor([2, 0], dtype=torch.int32, device=device), pos, offs)
    close(out[:43], want[40:], dtype, "continued segment")
    close(out[43:], want[:17], dtype, "fresh segment into a stale slot")


@pytest.mark.parametrize("device", DEVICES)
def test_grouped_routing(device):
    """Scores, correction for the choice only, the best groups, ties to the lower index, choice
    scores below zero (a masked group must not win against them), weights renormalised and scaled."""
    g = torch.Generator().manual_seed(7)
    for (T, E, k, groups, keep, scale) in ((50, 6, 3, 3, 2, 1.7), (33, 20, 4, 5, 3, 2.0), (20, 8, 2, 1, 1, 1.0),
                                           (40, 12, 3, 4, 1, 0.5), (9, 1, 1, 1, 1, 3.0), (25, 64, 8, 8, 4, 1.0)):
        z = 2.0 * torch.randn(T, E, generator=g)
        z[0, :] = 0.25                                        # all tied: the lowest indices of the lowest groups
        corr = torch.randn(E, generator=g) * 0.5 / E
        if E >= 6:
            corr[: E // groups] -= 2.0                        # a whole group far below zero
        r = {"top": k, "scale": scale}
        if groups > 1:
            r["groups"] = {"count": groups, "keep": keep}
        want = O.route(z.double(), corr, r)
        ids, wts = ops.moe_route_grouped(z.to(device), corr.to(device), k, groups, keep, scale)
        for t in range(T):
            assert ids[t].tolist() == [e for e, _ in want[t]], f"row {t}: experts chosen"
            close(wts[t], torch.tensor([w for _, w in want[t]]), "float32", "weights")
    with pytest.raises(ValueError):
        ops.moe_route_grouped(z.to(device), corr.to(device), 40, 8, 4, 1.0)


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_experts_with_identity_and_shared(device, dtype):
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(9)
    for (T, H, E, n_id, k, F) in ((33, 40, 5, 1, 3, 14), (70, 24, 3, 0, 2, 7), (150, 256, 4, 2, 2, 128), (12, 16, 1, 3, 2, 8)):
        x = torch.randn(T, H, generator=g).to(tdt)
        logits = torch.randn(T, E + n_id, generator=g)
        corr = torch.zeros(E + n_id)
        ids, wts = ops.moe_route_grouped(logits.to(device), corr.to(device), k, 1, 1, 1.3)
        w13 = (torch.randn(E, 2 * F, H, generator=g) * H ** -0.5).to(tdt)
        w2 = (torch.randn(E, H, F, generator=g) * F ** -0.5).to(tdt)
        add = torch.randn(T, H, generator=g).to(tdt)
        got = ops.moe_glu_experts(x.to(device), ids, wts, w13.to(device), w2.to(device), math.inf, 1.0, weight_input=False,
                                  add=add.to(device), shift=0.0, identity=n_id > 0)
        want = add.double().clone()
        xd = x.double()
        for t in range(T):
            for e, s in zip(ids[t].tolist(), wts[t].tolist()):
                if e >= E:
                    want[t] += s * xd[t]
                else:
                    hh = O.silu(xd[t] @ w13[e, :F].double().T) * (xd[t] @ w13[e, F:].double().T)
                    want[t] += s * (hh @ w2[e].double().T)
        assert n_id == 0 or bool((ids >= E).any()), "an identity expert is chosen somewhere"
        close(got, want, dtype, f"experts {E} + {n_id} identity, top {k}, ff {F}")


# ---------------------------------------------------------------------------- the model on the engine
@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_whole_prompt_and_layer_runs(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(200)
    runs = []
    want = O.forward(cd, W, toks, runs)
    tap = []
    got = eng.replay_step([(1, toks, list(range(len(toks))))], [1], layer_tap=tap)
    assert len(tap) == len(runs) == len(O.layer_runs(cd))
    for i, (a, b) in enumerate(zip(tap, runs)):
        close_rows(a, b, dtype, f"residual stream after run {i} (layer {O.layer_runs(cd)[i][0]})")
    close_rows(got, want, dtype, "logits")
    close_rows(got[:3], O.forward(cd, W, toks[:3]), dtype, "first tokens")
    close_rows(eng.replay_step([(2, toks[:1], [0])], [2]), O.forward(cd, W, toks[:1]), dtype, "a prompt of one token")


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_prefill_then_decode_and_portions(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(230, seed=5)
    want = O.forward(cd, W, toks)
    close_rows(replay_cuts(eng, toks, [70]), want, dtype, "prompt then token by token (160 decoded)")
    close_rows(replay_cuts(eng, toks, [1] * 3 + [2, 61, 2, 3, 64, 2, 63, 2, 17]), want, dtype, "portions down to two tokens")
    if shape == "odd":
        close_rows(replay_cuts(eng, toks, []), want, dtype, "token by token from the first")
    assert eng.sched.free_blocks() == eng.num_blocks


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_mixed_batches_and_reuse(device, dtype, shape):
    """Unequal requests interleaved (portions beside single tokens, a request that skips steps),
    in a pool that only holds the live ones: pages and state slots are freed and used again by
    requests that start later. Every request must equal its run alone (the oracle)."""
    eng, cd, W = build(device, dtype, pages=9, seqs=3, cd=CFGS[shape]())
    reqs = {i: tokens(n, seed=10 + i) for i, n in enumerate((150, 65, 1, 200, 129, 64, 3))}
    want = {i: O.forward(cd, W, t) for i, t in reqs.items()}
    got = {i: [] for i in reqs}
    at = {i: 0 for i in reqs}
    waiting, live, step = sorted(reqs), [], 0
    plans = {0: [64, 1, 1, 30], 1: [2, 62], 3: [100, 2], 4: [128], 5: [63]}
    while waiting or live:
        while waiting and len(live) < 3:
            nxt = waiting[0]
            need = sum(-(-len(reqs[i]) // 64) for i in live) + -(-len(reqs[nxt]) // 64)
            if need > 9:
                break
            live.append(waiting.pop(0))
        rows, fin = [], []
        for i in list(live):
            if i == 3 and step % 3 == 1:
                continue                                  # left out of this step, goes on later
            plan = plans.get(i, [])
            n = min(plan.pop(0) if plan else 1, len(reqs[i]) - at[i])
            rows.append((100 + i, reqs[i][at[i]:at[i] + n], list(range(n))))
            at[i] += n
            if at[i] == len(reqs[i]):
                fin.append(100 + i)
                live.remove(i)
        lg = eng.replay_step(rows, fin)
        k = 0
        for rid, t, _ in rows:
            got[rid - 100].append(lg[k:k + len(t)])
            k += len(t)
        step += 1
    for i in reqs:
        close_rows(torch.cat(got[i]), want[i], dtype, f"request {i} in the batch")
    assert eng.sched.free_blocks() == 9 and eng.sched.free_state_slots() == 3


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_sizes_that_coincide_elsewhere(device, dtype):
    """One head, one kv head per head and one for all, one expert with top 1, only identity
    choices possible beside it, a rotation of one pair and of the whole head, vdim = dim, no cap,
    no loop, a loop of one pass over everything, layers without feed-forward first and last, a
    width that is no multiple of 8."""
    layers = [att(heads=1, kv=1, dim=2, vdim=3, dims=2), mlstm(heads=1, dim=1, vdim=1, cap=1.0, mlp=moe(1, 1, 8, 0, None, 1.0, None)),
              att2(heads=6, kv=1, dim=4, dims=4, cap=0.0, scaling=None, mlp=moe(1, 2, 5, 3, (2, 1), 0.7, 3)),
              mlstm(heads=4, dim=6, vdim=6, cap=30.0, mlp=dense(6)), att(heads=2, kv=2, dim=6, vdim=6, dims=6)]
    toks = tokens(140, vocab=61, seed=9)
    for loop in (None, (0, 5, 1), (4, 5, 3)):
        cd = cfg_dict(layers, width=36, vocab=61, loop=loop)
        eng, cd, W = build(device, dtype, cd=cd)
        close_rows(replay_cuts(eng, toks, [66, 5]), O.forward(cd, W, toks), dtype, f"odd sizes, loop {loop}")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_long_decoding(device, dtype):
    """300 tokens decoded one by one after a short prompt: the recurrent state and its running
    maximum carried through hundreds of single-row steps, rotations at growing positions, pages
    filled and crossed by decoded tokens only."""
    cd = cfg_dict([mlstm(mlp=moe()), att2(mlp=dense()), att()], loop=(0, 2, 2))
    eng, cd, W = build(device, dtype, cd=cd)
    toks = tokens(330, seed=6)
    close_rows(replay_cuts(eng, toks, [30]), O.forward(cd, W, toks), dtype, "long decoding")


@pytest.mark.parametrize("device,dtype", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_scheduler(device, dtype):
    """LLMEngine.generate: the engine's own scheduler chunks the prompts (a small token budget),
    batches the requests and decodes (hipGraph decode steps on the GPU); greedy tokens must
    equal the oracle's."""
    eng, cd, W = build(device, dtype, pages=16, max_batched_tokens=48, token_alignment=1, mixed_prefill_tokens=16)
    prompts = [tokens(90, seed=21), tokens(5, seed=22), tokens(67, seed=23)]
    reqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, r in zip(prompts, reqs):
        assert r.output_ids == O.greedy(cd, W, p, 12)
    assert eng.stats["prefill_steps"] > 2 and eng.sched.free_blocks() == 16


@pytest.mark.parametrize("device", DEVICES)
def test_pipelined_generation_matches_synchronous(device):
    a, cd, W = build(device, "float32", async_decode=True)
    b, _, _ = build(device, "float32", async_decode=False)
    prompts = [tokens(40, seed=31), tokens(70, seed=32)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    assert [r.output_ids for r in a.generate(prompts, sp)] == [r.output_ids for r in b.generate(prompts, sp)]


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_recomputes(device):
    """A pool too small for both sequences to grow: the scheduler preempts one (its pages and
    state slot go back), recomputes it later from its first token, and the tokens do not change."""
    small, cd, W = build(device, "float32", pages=5)
    big, _, _ = build(device, "float32", pages=16)
    prompts = [tokens(120, seed=41), tokens(120, seed=42)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    got = [r.output_ids for r in small.generate(prompts, sp)]
    assert small.sched.preemptions() > 0
    assert got == [r.output_ids for r in big.generate(prompts, sp)]
    assert got[0] == O.greedy(cd, W, prompts[0], 20)
    assert small.sched.free_blocks() == 5


def test_model_folder_roundtrip(tmp_path):
    """config.json + safetensors -> registry -> engine (EngineConfig.model as a folder)."""
    from nv_genai_amd.models.registry import read_config
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_odd()
    cfg = LizezenConfig.from_dict(cd)
    assert cfg.to_json_dict() == cd
    assert cfg.is_moe and cfg.experts_per_tok == 3 and cfg.num_experts == 5
    assert [li for li, _ in cfg.runs] == [0, 1, 2, 3, 1, 2, 3, 4] and [f for _, f in cfg.runs] == [False, True, False, False,
                                                                                                 True, False, False, False]
    w = random_weights(cfg, 3, torch.bfloat16)
    save_weights(w, str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(cd))
    got, cls = read_config(str(tmp_path))
    assert cls is LizezenModel and got == cfg
    eng = LLMEngine(EngineConfig(model=str(tmp_path), dtype="float32", max_num_seqs=2, max_batched_tokens=128,
                                 max_model_len=128, kv_cache_blocks=4, detokenize=False, use_graphs=False,
                                 mixed_graphs=False, tuned_gemms=False, async_decode=False), device="cpu")
    toks = tokens(50, seed=7)
    close_rows(eng.replay_step([(1, toks, list(range(50)))], [1]), O.forward(cd, w, toks), "float32", "model folder")
    sd = eng.model.state_dict()
    assert set(sd) == set(w)
    for k in w:
        assert torch.equal(sd[k].cpu().reshape(w[k].shape).to(w[k].dtype), w[k]), k


def test_config_errors_and_builder():
    bad = cfg_odd()
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(bad)
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(cfg_dict([att(mlp=moe(3, 5, 7, 0, None))]))   # top above the experts
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(cfg_dict([att(mlp=moe(5, 3, 7, 0, (3, 2)))]))  # groups do not divide the experts
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(cfg_dict([att(dim=4, dims=6)]))               # rotation longer than the head
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(cfg_dict([att(heads=5, kv=2)]))
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(cfg_dict([att(mlp={"kind": "conv"})]))
    with pytest.raises(ValueError):
        LizezenConfig.from_dict(cfg_dict([att()], loop=(0, 2, 2)))            # the span ends behind the last layer
    cfg = LizezenConfig.from_dict(cfg_odd())
    w = random_weights(cfg, 0)
    w["l0.mix.norm"] = w["l0.mix.norm"][:-1]
    with pytest.raises(ValueError):
        LizezenModel(cfg, "cpu", torch.float32, weights=w)
    c = lizezen_layers(["mlstm", "attention", "attention_2", "mlstm"], 64, 4, 2, 16, 8, 48, mlstm_heads=2, mlstm_dim=8,
                       mlstm_vdim=16, experts=4, top=2, expert_ff=16, shared_ff=8, identity=2, groups=3, keep=2,
                       route_scale=2.0, softcap=12.0, yarn=(4.0, 64, 8.0, 1.0), loop=(1, 3, 2))
    assert c.blocks[2].mixer.rot.yarn and not c.blocks[1].mixer.rot.yarn and c.blocks[2].mixer.values_from_keys
    assert LizezenConfig.from_dict(c.to_json_dict()) == c
    assert len(c.runs) == 6


@pytest.mark.gpu
def test_mfma_forms_run_and_agree_with_the_plain_kernels():
    """At layer sizes (bf16): the engine's attention choice, capped scores and the head gate on the
    MFMA prompt and single-token kernels against the row kernel, and the grouped MFMA SwiGLU expert
    GEMMs with identity experts against the tiled fp32-accumulating ones."""
    dev = "cuda"
    g = torch.Generator().manual_seed(2)
    q = torch.randn(4, 128 * 8, generator=g).bfloat16().to(dev)
    assert ops.softmax_attention_mfma_ok(q, 128, 128, 4, 1) and ops.softmax_attention_mfma_ok(q, 64, 64, 1, 1)
    assert not ops.softmax_attention_mfma_ok(q, 96, 96, 1, 1)
    H, G, dk, dv, npg, cap = 8, 2, 128, 128, 40, 1.5
    kc = (0.5 * torch.randn(npg, G, 64, dk, generator=g)).bfloat16().to(dev)
    vc = torch.randn(npg, G, 64, dv, generator=g).bfloat16().to(dev)
    bt = torch.randperm(npg, generator=g).to(torch.int32).view(2, 20).to(dev)
    cu = torch.tensor([0, 301, 370], dtype=torch.int32, device=dev)
    ctx = torch.tensor([1000, 69], dtype=torch.int32, device=dev)
    qq = (2.0 * torch.randn(370, H * dk, generator=g)).bfloat16().to(dev)
    gate = torch.randn(370, H, generator=g).bfloat16().to(dev)
    seq, pos = ops._rows_of_portions(cu, ctx, 370, dev)
    kw = dict(scale=dk ** -0.5, softcap=cap, gate=gate)
    want = ops.softmax_attention(qq, kc, vc, bt, seq, pos, H, G, dk, dv, **kw).float()
    free = ops.softmax_attention(qq, kc, vc, bt, seq, pos, H, G, dk, dv, scale=dk ** -0.5, gate=gate).float()
    assert (want - free).abs().max().item() > 0.1, "the cap changes the result at these scores"
    got = ops.softmax_attention_prefill(qq, kc, vc, bt, cu, ctx, 301, H, G, dk, dv, **kw).float()
    assert (got - want).abs().max().item() < 0.03 * max(1.0, want.abs().max().item())
    got = ops.softmax_attention_rows(qq, kc, vc, bt, seq, pos, H, G, dk, dv, max_ctx=1024, **kw).float()
    assert (got - want).abs().max().item() < 0.03 * max(1.0, want.abs().max().item())
    T, W, E, k, F = 700, 512, 8, 3, 256
    x = torch.randn(T, W, generator=g).bfloat16().to(dev)
    w13 = (torch.randn(E, 2 * F, W, generator=g) * W ** -0.5).bfloat16().to(dev)
    w2 = (torch.randn(E, W, F, generator=g) * F ** -0.5).bfloat16().to(dev)
    ids, wts = ops.moe_route_grouped(torch.randn(T, E + 2, generator=g).to(dev), torch.zeros(E + 2, device=dev), k, 2, 2, 2.0)
    assert ops.moe_mfma_ok(x, F)
    a = ops.moe_glu_experts(x, ids, wts, w13, w2, math.inf, 1.0, False, shift=0.0, identity=True).float()
    b = ops.moe_glu_experts(x.float(), ids, wts, w13.float(), w2.float(), math.inf, 1.0, False, shift=0.0, identity=True)
    assert (a - b).abs().max().item() < 0.03 * max(1.0, b.abs().max().item())


@pytest.mark.parametrize("device", DEVICES)
def test_trace_runner_replays_a_schedule(device, tmp_path, monkeypatch, capsys):
    """The trace runner on a model folder: steps as JSON lines on standard input (a prompt in two
    portions, a second request beside single tokens of the first, requests ended and their names
    used again), logits files of the wanted places, a ``done`` line per step."""
    import io

    import numpy as np

    from nv_genai_amd.tools import trace_run
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_dict([mlstm(mlp=moe()), att2(mlp=dense()), att()], loop=(1, 3, 2))
    cfg = LizezenConfig.from_dict(cd)
    w = random_weights(cfg, 8, torch.bfloat16)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    save_weights(w, str(model_dir))
    (model_dir / "config.json").write_text(json.dumps(cd))
    a, b = tokens(80, seed=51), tokens(30, seed=52)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:65], "want": [0, 64]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[65:78], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[:29], "want": [28]}, {"id": "a", "tokens": a[78:79], "want": [0]}],
              "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[79:], "want": [0]}, {"id": "b", "tokens": b[29:], "want": [0]}],
              "end": ["a", "b"]},
             {"step": 4, "entries": [{"id": "a", "tokens": b[:5], "want": [4]}], "end": ["a"]}]
    monkeypatch.setattr("sys.stdin", io.StringIO("".join(json.dumps(s) + "\n" for s in steps)))
    rc = trace_run.main(["--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir), "--max-tokens", "192",
                         "--device", device])
    assert rc == 0
    assert [l for l in capsys.readouterr().out.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    wa, wb = O.forward(cd, w, a), O.forward(cd, w, b)
    V = cd["vocab"]

    def rows(i):
        return torch.from_numpy(np.fromfile(out_dir / f"{i}.f32", dtype="<f4").reshape(-1, V).copy())

    assert not (out_dir / "1.f32").exists()
    close_rows(rows(0), wa[[0, 64]], "float32", "first portion")
    close_rows(rows(2), torch.stack([wb[28], wa[78]]), "float32", "a portion beside a single token")
    close_rows(rows(3), torch.stack([wa[79], wb[29]]), "float32", "last tokens")
    close_rows(rows(4), wb[4:5], "float32", "a name used again")
