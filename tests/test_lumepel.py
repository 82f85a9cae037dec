"""Lumepel on the serving engine against the plain oracle (tests/lumepel_oracle.py).

Every case runs on the CPU (the engine on the fp32 reference ops: scheduling, pages, row maps)
and, marked ``gpu``, on the HIP kernels in float32 and bfloat16. The models are small random ones
built here; sizes are chosen so that heads, dims, ranks, expert counts and the page size do not
coincide (``odd``: rotation on fewer elements than the rotated part, top-2 of 5 and top-3 of 3
experts, a layer without a shared expert, one without feed-forward), or so that the MFMA tile
kernels run (``tiles``).
"""
import json
import math

import pytest
import torch

import lumepel_oracle as O
from nv_genai_amd import ops
from nv_genai_amd.engine.llm_engine import EngineConfig, LLMEngine, SamplingParams
from nv_genai_amd.models.config import LumepelConfig, lumepel_layers
from nv_genai_amd.models.lumepel import GLU_ALPHA, LumepelModel, random_weights

GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVICES = ["cpu", GPU]
DTYPES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
          pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}


def dense(ff=24, limit=0.6):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=5, top=2, ff=24, limit=0.8, shared=(12, 1.2)):
    d = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


def lat(heads=3, dim=8, rot_dim=6, dims=4, vdim=12, kv_rank=20, q_rank=10, scale=0.3, base=100.0, scaling=YARN,
        mlp=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(scaling)
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                      "q_rank": q_rank, "scale": scale, "rot": rot}, "mlp": mlp}


def lat2(heads=5, dim=4, rot_dim=8, dims=8, vdim=4, kv_rank=9, scale=0.25, base=50.0, mlp=None):
    return {"type": "latent_attention_2",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": dims}}, "mlp": mlp}


def cfg_dict(layers, width=40, vocab=97, eps=1e-5, scale=7.0, cap=25.0, logit_scale=0.7):
    return {"architecture": "Lumepel", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "logit_scale": logit_scale, "logit_softcap": cap, "layers": layers}


def cfg_odd():
    return cfg_dict([lat(mlp=moe()), lat2(mlp=dense()),
                     lat(heads=2, dim=12, rot_dim=4, dims=4, vdim=8, kv_rank=33, q_rank=7, scaling=None),
                     lat2(heads=1, dim=6, rot_dim=2, dims=2, vdim=10, kv_rank=5, mlp=moe(3, 3, 7, 2.0, None))])


def cfg_tiles():
    """Sizes the MFMA kernels take: latent + rotated part of 64 + 32 and 128 + 64 elements, 18 heads
    over one latent, experts of 128 on a width of 256."""
    return cfg_dict([lat(heads=18, dim=16, rot_dim=32, dims=32, vdim=16, kv_rank=64, q_rank=24, scale=0.15,
                         base=10000.0, scaling={"factor": 8.0, "original": 64, "fast": 16.0, "slow": 1.0},
                         mlp=moe(4, 2, 128, 1.0, (64, 1.5))),
                     lat2(heads=4, dim=32, rot_dim=64, dims=64, vdim=32, kv_rank=128, scale=0.1, base=1000.0,
                          mlp=dense(64, 1.0))], width=256)


CFGS = {"odd": cfg_odd, "tiles": cfg_tiles}


def build(device, dtype="float32", seed=0, pages=24, seqs=4, cd=None, graphs=None, **eng):
    cd = cd or cfg_odd()
    cfg = LumepelConfig.from_dict(cd)
    w = random_weights(cfg, seed, torch.bfloat16)       # bf16 values, as a checkpoint holds them
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    model = LumepelModel(cfg, device, tdt, weights=w)
    kw = dict(model="lumepel-test", dtype=dtype, max_num_seqs=seqs, max_batched_tokens=512, max_model_len=512,
              kv_cache_blocks=pages, detokenize=False, use_graphs=(device == "cuda") if graphs is None else graphs,
              graph_batch_sizes=(1, 2, 4), mixed_graphs=False, logits_tap=True, tuned_gemms=False, async_decode=False,
              enable_prefix_caching=False)   # replayed rows bring every token themselves
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
def test_rotary_frequencies_plain_and_scaled():
    for rot in ({"dims": 8, "base": 50.0}, {"dims": 32, "base": 1e4, "scaling": {"factor": 8.0, "original": 64,
                                                                              "fast": 16.0, "slow": 1.0}},
                {"dims": 4, "base": 100.0, "scaling": YARN}, {"dims": 64, "base": 1e6, "scaling": {
                    "factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}}):
        sc = rot.get("scaling")
        f, mag = ops.rotary_frequencies(rot["dims"], rot["base"],
                                        None if not sc else (sc["factor"], sc["original"], sc["fast"], sc["slow"]))
        fo, mo = O.rope_frequencies(rot)
        assert torch.allclose(f, fo, rtol=1e-14, atol=0) and abs(mag - mo) < 1e-15
        if sc:   # the fastest pair is untouched, the slowest divided by the factor
            assert f[0] == 1.0 and abs(float(f[-1]) * sc["factor"] / rot["base"] ** (-(rot["dims"] - 2) / rot["dims"]) - 1) < 1e-12


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_stream_ops_glu_softcap(device, dtype):
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(3)
    T, H, F = 37, 41, 23
    x0 = torch.randn(T, H, generator=g)
    y = torch.randn(T, H, generator=g).to(tdt)
    w = 1.0 + 0.2 * torch.randn(H, generator=g)
    x = x0.clone().to(device)
    h = ops.residual_add_rmsnorm_(x, y.to(device), w.to(device), 1e-5, tdt)
    xs = x0.double() + y.double()
    close(x, xs, "float32", "residual sum stays fp32")
    close(h, O.rmsnorm(xs, w.double(), 1e-5), dtype, "norm of the sum")
    assert ops.residual_add_rmsnorm_(x, y.to(device), None, 1e-5, tdt) is None
    close(x, xs + y.double(), "float32", "sum only")
    # clamped GLU: values on both sides of the limits, a gate column behind padding; widths the
    # 8-wide form takes and widths it does not
    for F, pad, lim in ((23, 3, 0.5), (23, 3, 7.0), (24, 8, 0.5), (24, 8, 7.0)):
        gu = (3.0 * torch.randn(T, 2 * F + pad, generator=g)).to(tdt)
        a = ops.clamped_glu(gu.to(device), F, lim, GLU_ALPHA)
        gg, uu = gu[:, :F].double().clamp(max=lim), gu[:, F:2 * F].double().clamp(-lim, lim)
        want = gg * torch.sigmoid(1.702 * gg) * (uu + 1.0)
        close(a, want, dtype, f"clamped glu limit {lim}")
        a = ops.clamped_glu(gu.to(device), F, lim, GLU_ALPHA, gate_col=2 * F + 1)
        close(a, want * torch.sigmoid(gu[:, 2 * F + 1:2 * F + 2].double()), dtype, "row gate")
    z = (40.0 * torch.randn(T, 50, generator=g))
    close(ops.scale_softcap_(z.clone().to(device), 0.5, 30.0), 30.0 * torch.tanh(z.double() * 0.5 / 30.0), "float32", "cap")
    close(ops.scale_softcap_(z.clone().to(device), 2.0, 0.0), z.double() * 2.0, "float32", "scale without a cap")


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_latent_norm_rotation_and_page_write(device, dtype, interleaved):
    """Positions far out (the angle must stay exact), a rotation on fewer elements than the rotated
    part, slots in several pages, a row that is not written."""
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(5)
    T, Hh, d, dr, dims, r, nq = 9, 3, 5, 8, 6, 11, 7
    rot = {"dims": dims, "base": 30.0, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}
    freq, mag = ops.rotary_frequencies(dims, 30.0, (4.0, 16, 4.0, 1.0))
    W = r + dr
    cols = nq + Hh * (d + dr) + r + dr + 2
    proj0 = torch.randn(T, cols, generator=g).to(tdt)
    pos = torch.tensor([0, 1, 63, 64, 1000, 65535, 99999, 7, 2], dtype=torch.int32)
    slots = torch.tensor([0, 1, 63, 64, 130, 191, 5, -1, 70], dtype=torch.int32)
    nw, cw = 1 + 0.1 * torch.randn(nq, generator=g), 1 + 0.1 * torch.randn(r, generator=g)
    page = torch.zeros(3, 1, 64, W, dtype=tdt, device=device)
    q_out = torch.zeros(T, Hh * W, dtype=tdt, device=device)
    proj = proj0.clone().to(device)
    q_off, kv_off = nq, nq + Hh * (d + dr)
    ops.latent_rope_cache_(proj, pos.to(device), slots.to(device), page, freq.to(device), mag, interleaved, dims, dr, 1e-5,
                           kv=(kv_off, r, cw.to(device)), q=(q_off, Hh, d), q_out=q_out, norm=(0, nq, nw.to(device)))
    pd = proj0.double()
    close(proj[:, :nq], O.rmsnorm(pd[:, :nq], nw.double(), 1e-5), dtype, "in-place norm")
    assert torch.equal(proj[:, nq:].cpu(), proj0[:, nq:]), "the other columns stay"
    c = O.rmsnorm(pd[:, kv_off:kv_off + r], cw.double(), 1e-5)
    kr = O.rotate(pd[:, kv_off + r:kv_off + r + dr], pos, rot, interleaved)
    qr = O.rotate(pd[:, q_off:kv_off].view(T, Hh, d + dr)[:, :, d:], pos, rot, interleaved)
    close(q_out.view(T, Hh, W)[:, :, r:], qr, dtype, "rotated query parts")
    assert float(q_out.view(T, Hh, W)[:, :, :r].abs().max()) == 0.0
    rows = page.view(-1, W)
    for t in range(T):
        if slots[t] >= 0:
            close(rows[int(slots[t])], torch.cat([c[t], kr[t]]), dtype, f"page row of token {t}")
    written = torch.zeros(192, dtype=torch.bool)
    written[slots[slots >= 0].long()] = True
    assert float(rows[~written.to(rows.device)].abs().max()) == 0.0


def _latent_page(c, device, tdt, bt_row, nb):
    """Token rows c [n, W] laid into pages [nb, 1, 64, W] through the block-table row."""
    n, W = c.shape
    page = torch.zeros(nb, 1, 64, W, dtype=tdt, device=device)
    j = torch.arange(n)
    page[bt_row[j // 64].long(), 0, j % 64] = c.to(tdt).to(device)
    return page


def o_attention_in_keys(q, rows, dv, scale, pos):
    """Plain form: query t at position pos[t] sees key rows 0 .. pos[t]; values = first dv columns."""
    T, H, W = q.shape
    out = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        k = rows[: int(pos[t]) + 1].double()
        a = torch.softmax(q[t].double() @ k.T * scale, -1)
        out[t] = a @ k[:, :dv]
    return out.reshape(T, H * dv)


@pytest.mark.parametrize("shape", [(3, 26, 20), (18, 96, 64), (4, 192, 128), (2, 320, 256), (1, 13, 13), (2, 64, 32),
                                   (3, 128, 64), (2, 256, 128), (1, 600, 530), (3, 96, 64)])
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_one_key_stands_out_and_random(device, dtype, shape):
    """Values read out of the key rows. One key row is made to match a scaled query, far back,
    on both sides of page borders, at the query's own position, and one position *after* the query
    (it must not be seen): the output is that key's leading columns or not. Through the row kernel,
    the prompt kernel (one portion) and the single-token kernel."""
    H, W, dv = shape
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(11)
    n = 700
    rows = (0.3 * torch.randn(n, W, generator=g)).to(tdt).float()
    bt = torch.randperm(16, generator=g)[:11].to(torch.int32)
    qpos = [699, 640, 128, 127, 64, 63, 5, 0]
    marks = [3, 63, 64, 127, 128, 575, 576, 639]
    scale = W ** -0.5
    for hot in marks + [None]:
        R = rows.clone()
        u = torch.randn(W, generator=g)
        u = u / u.norm()
        if hot is not None:
            R[hot] = (6.0 * u).to(tdt).float()
        page = _latent_page(R, device, tdt, bt, 16)
        q = (0.3 * torch.randn(len(qpos), H, W, generator=g))
        if hot is not None:
            q[:, 0] = 40.0 * u / scale / 6.0      # head 0: score 40 on the hot key
        q = q.to(tdt)
        pos = torch.tensor(qpos, dtype=torch.int32)
        want = o_attention_in_keys(q.float(), R, dv, scale, pos)
        qd = q.reshape(len(qpos), H * W).to(device)
        seq = torch.zeros(len(qpos), dtype=torch.int32, device=device)
        btd = bt.view(1, -1).to(device)
        kw = dict(scale=scale, v_in_k=True)
        got = ops.softmax_attention(qd, page, page, btd, seq, pos.to(device), H, 1, W, dv, **kw)
        close(got, want, dtype, f"row form, hot key {hot}")
        got = ops.softmax_attention_rows(qd, page, page, btd, seq, pos.to(device), H, 1, W, dv, max_ctx=704, **kw)
        close(got, want, dtype, f"single-token form, hot key {hot}")
        if hot is not None:
            for t, p in enumerate(qpos):
                hit = (got[t, :dv].double().cpu() - R[hot, :dv].double()).abs().max().item() < 0.05
                assert hit == (hot <= p), f"query at {p}, hot key at {hot}: seen={hit}"
    # a portion: queries at positions 560 .. 699 of the same sequence in one launch
    R = rows.clone()
    u = torch.randn(W, generator=g)
    u = u / u.norm()
    R[600] = (6.0 * u).to(tdt).float()
    page = _latent_page(R, device, tdt, bt, 16)
    nq = 140
    q = 0.3 * torch.randn(nq, H, W, generator=g)
    q[:, H - 1] = 40.0 * u / scale / 6.0
    q = q.to(tdt)
    pos = torch.arange(560, 700, dtype=torch.int32)
    want = o_attention_in_keys(q.float(), R, dv, scale, pos)
    cu = torch.tensor([0, nq], dtype=torch.int32, device=device)
    ctx = torch.tensor([700], dtype=torch.int32, device=device)
    got = ops.softmax_attention_prefill(q.reshape(nq, H * W).to(device), page, page, bt.view(1, -1).to(device), cu, ctx, nq,
                                        H, 1, W, dv, scale=scale, v_in_k=True)
    close(got, want, dtype, "portion")
    for t in (39, 40, 41):     # positions 599 (the key comes one later), 600, 601
        hit = (got[t, (H - 1) * dv:].double().cpu() - R[600, :dv].double()).abs().max().item() < 0.05
        assert hit == (t >= 40)


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_routing_and_experts(device, dtype):
    tdt = tdtype(dtype)
    g = torch.Generator().manual_seed(7)
    for (T, H, E, k, F, lim, width_in) in ((33, 40, 5, 2, 24, 0.8, True), (70, 24, 3, 3, 7, 2.0, True),
                                           (5, 16, 9, 1, 16, 0.4, False), (150, 256, 4, 2, 128, 1.0, True)):
        x = torch.randn(T, H, generator=g).to(tdt)
        router = torch.randn(E, H, generator=g) * H ** -0.5
        logits = x.float() @ router.T
        logits[0, :] = 0.25                                  # a row of ties: the lowest indices win
        ids, wts = ops.moe_route_scores(logits.to(device), k, "sigmoid", False)
        oi, ow = O.route(x.double(), router.double(), k)
        oi[0], ow[0] = torch.arange(k), torch.sigmoid(torch.tensor(0.25, dtype=torch.float64))
        assert torch.equal(ids.cpu().long(), oi), "experts chosen"
        close(wts, ow, "float32", "weights are the scores as they are")
        _, wn = ops.moe_route_scores(logits.to(device), k, "softmax", True)
        ps = torch.softmax(logits.double(), -1).gather(1, oi)
        close(wn, ps / ps.sum(-1, keepdim=True), "float32", "softmax scores renormalised")
        w13 = (torch.randn(E, 2 * F, H, generator=g) * H ** -0.5).to(tdt)
        w2 = (torch.randn(E, H, F, generator=g) * F ** -0.5).to(tdt)
        add = torch.randn(T, H, generator=g).to(tdt)
        got = ops.moe_glu_experts(x.to(device), ids, wts, w13.to(device), w2.to(device), lim, GLU_ALPHA,
                                  weight_input=width_in, add=add.to(device))
        want = add.double().clone()
        for t in range(T):
            for e, s in zip(oi[t].tolist(), ow[t].tolist()):
                hin = x[t:t + 1].double() * (s if width_in else 1.0)
                y = O.clamped_glu(hin, w13[e, :F].double(), w13[e, F:].double(), w2[e].double(), lim)[0]
                want[t] += y if width_in else y * s
        close(got, want, dtype, f"experts {E} top {k} ff {F}")


# ---------------------------------------------------------------------------- the model on the engine
@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_whole_prompt_and_layers(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(200)
    layers = []
    want = O.forward(cd, W, toks, layers)
    tap = []
    got = eng.replay_step([(1, toks, list(range(len(toks))))], [1], layer_tap=tap)
    for i, (a, b) in enumerate(zip(tap, layers)):
        close(a, b, dtype, f"residual stream after layer {i} ({cd['layers'][i]['type']})")
    close(got, want, dtype, "logits")
    close(got[:3], O.forward(cd, W, toks[:3]), dtype, "first tokens")
    close(eng.replay_step([(2, toks[:1], [0])], [2]), O.forward(cd, W, toks[:1]), dtype, "a prompt of one token")


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_prefill_then_decode_and_portions(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(230, seed=5)
    want = O.forward(cd, W, toks)
    close(replay_cuts(eng, toks, [70]), want, dtype, "prompt then token by token (160 decoded)")
    close(replay_cuts(eng, toks, [1] * 3 + [2, 61, 2, 3, 64, 2, 63, 2, 17]), want, dtype, "portions down to two tokens")
    if shape == "odd":
        close(replay_cuts(eng, toks, []), want, dtype, "token by token from the first")
    assert eng.sched.free_blocks() == eng.num_blocks


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_mixed_batches_and_reuse(device, dtype, shape):
    """Unequal requests interleaved (portions beside single tokens, a request that skips steps),
    in a pool that only holds the live ones: pages and slots are freed and used again by requests
    that start later. Every request must equal its run alone (the oracle)."""
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
        close(torch.cat(got[i]), want[i], dtype, f"request {i} in the batch")
    assert eng.sched.free_blocks() == 9 and eng.sched.free_state_slots() == 3


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_sizes_that_coincide_elsewhere(device, dtype):
    """One head, one expert with top 1, a latent wider than the model, a rotation of one pair, a
    rotated part as long as the unrotated one, no cap and no logit scale, dim = vdim = rot_dim,
    layers without feed-forward first and last, a width that is no multiple of 8."""
    cd = cfg_dict([lat2(heads=1, dim=4, rot_dim=2, dims=2, vdim=4, kv_rank=50),
                   lat(heads=1, dim=6, rot_dim=6, dims=6, vdim=6, kv_rank=6, q_rank=60, scaling=None,
                       mlp=moe(1, 1, 8, 1.0, None)),
                   lat2(heads=6, dim=12, rot_dim=12, dims=12, vdim=12, kv_rank=8, mlp=moe(2, 1, 5, 0.3, (3, 0.2))),
                   lat(heads=2, dim=2, rot_dim=10, dims=2, vdim=1, kv_rank=3, q_rank=1)], width=36, vocab=61, cap=0.0,
                  scale=1.0, logit_scale=1.0)
    eng, cd, W = build(device, dtype, cd=cd)
    toks = tokens(140, vocab=61, seed=9)
    want = O.forward(cd, W, toks)
    close(replay_cuts(eng, toks, [66, 5]), want, dtype, "odd sizes")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_long_decoding(device, dtype):
    """300 tokens decoded one by one after a short prompt: rotations at growing positions, pages
    filled and crossed by decoded tokens only."""
    cd = cfg_dict([lat(mlp=moe()), lat2(mlp=dense())])
    eng, cd, W = build(device, dtype, cd=cd)
    toks = tokens(330, seed=6)
    close(replay_cuts(eng, toks, [30]), O.forward(cd, W, toks), dtype, "long decoding")


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
    """A pool too small for both sequences to grow: the scheduler preempts one (its pages go
    back), recomputes it later from its first token, and the tokens do not change."""
    small, cd, W = build(device, "float32", pages=5)
    big, _, _ = build(device, "float32", pages=16)
    prompts = [tokens(120, seed=41), tokens(120, seed=42)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    got = [r.output_ids for r in small.generate(prompts, sp)]
    assert small.sched.preemptions() > 0
    assert got == [r.output_ids for r in big.generate(prompts, sp)]
    assert got[0] == O.greedy(cd, W, prompts[0], 20)
    assert small.sched.free_blocks() == 5


@pytest.mark.parametrize("device", DEVICES)
def test_prefix_cache_reuses_pages(device):
    """A second request that starts with an earlier prompt takes its full pages from the prefix
    cache (only the rest is prefilled) and generates what the oracle generates."""
    eng, cd, W = build(device, "float32", enable_prefix_caching=True)
    p = tokens(150, seed=3)
    sp = SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)
    assert eng.generate([p], sp)[0].output_ids == O.greedy(cd, W, p, 8)
    before = eng.stats["prefill_tokens"]
    assert eng.generate([p + [5, 6, 7]], sp)[0].output_ids == O.greedy(cd, W, p + [5, 6, 7], 8)
    assert eng.stats["prefill_tokens"] - before == 153 - 128 and eng.sched.prefix_hits() > 0


def test_model_folder_roundtrip(tmp_path):
    """config.json + safetensors -> registry -> engine (EngineConfig.model as a folder)."""
    from nv_genai_amd.models.registry import read_config
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_odd()
    cfg = LumepelConfig.from_dict(cd)
    assert cfg.to_json_dict() == cd
    assert cfg.is_moe and cfg.experts_per_tok == 3 and cfg.num_experts == 5
    w = random_weights(cfg, 3, torch.bfloat16)
    save_weights(w, str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(cd))
    got, cls = read_config(str(tmp_path))
    assert cls is LumepelModel and got == cfg
    eng = LLMEngine(EngineConfig(model=str(tmp_path), dtype="float32", max_num_seqs=2, max_batched_tokens=128,
                                 max_model_len=128, kv_cache_blocks=4, detokenize=False, use_graphs=False,
                                 mixed_graphs=False, tuned_gemms=False, async_decode=False), device="cpu")
    toks = tokens(50, seed=7)
    close(eng.replay_step([(1, toks, list(range(50)))], [1]), O.forward(cd, w, toks), "float32", "model folder")
    sd = eng.model.state_dict()
    assert set(sd) == set(w)
    for k in w:
        assert torch.equal(sd[k].cpu().reshape(w[k].shape).to(w[k].dtype), w[k]), k


def test_config_errors_and_builder():
    bad = cfg_odd()
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        LumepelConfig.from_dict(bad)
    with pytest.raises(ValueError):
        LumepelConfig.from_dict(cfg_dict([lat(mlp=moe(3, 4))]))       # top above the experts
    with pytest.raises(ValueError):
        LumepelConfig.from_dict(cfg_dict([lat2(rot_dim=4, dims=6)]))  # rotation longer than the rotated part
    with pytest.raises(ValueError):
        LumepelConfig.from_dict(cfg_dict([lat(mlp={"kind": "conv"})]))
    cfg = LumepelConfig.from_dict(cfg_odd())
    w = random_weights(cfg, 0)
    w["l0.mix.dkv.norm"] = w["l0.mix.dkv.norm"][:-1]
    with pytest.raises(ValueError):
        LumepelModel(cfg, "cpu", torch.float32, weights=w)
    c = lumepel_layers(["latent_attention", "latent_attention_2"], 64, 4, 8, 4, 8, 16, 12, 0, experts=4, top=2,
                       expert_ff=16, shared_ff=8, yarn=(4.0, 64, 8.0, 1.0))
    assert c.blocks[0].mixer.q_rank == 12 and c.blocks[1].mixer.q_rank == 0 and c.blocks[0].mixer.rot.yarn
    assert LumepelConfig.from_dict(c.to_json_dict()) == c
    n = sum(t.numel() for t in random_weights(c, 0).values())
    assert n == c.num_params()


@pytest.mark.gpu
def test_mfma_forms_run_and_agree_with_the_plain_kernels():
    """At layer sizes (bf16): the grouped MFMA expert GEMMs against the tiled fp32-accumulating
    ones, and the engine's attention choice (MFMA where the sizes fit)."""
    dev = "cuda"
    g = torch.Generator().manual_seed(2)
    T, H, E, k, F = 700, 512, 8, 2, 256
    x = torch.randn(T, H, generator=g).bfloat16().to(dev)
    w13 = (torch.randn(E, 2 * F, H, generator=g) * H ** -0.5).bfloat16().to(dev)
    w2 = (torch.randn(E, H, F, generator=g) * F ** -0.5).bfloat16().to(dev)
    logits = torch.randn(T, E, generator=g).to(dev)
    ids, wts = ops.moe_route_scores(logits, k)
    assert ops.moe_mfma_ok(x, F)
    a = ops.moe_glu_experts(x, ids, wts, w13, w2, 1.0, GLU_ALPHA, True).float()
    b = ops.moe_glu_experts(x.float(), ids, wts, w13.float(), w2.float(), 1.0, GLU_ALPHA, True)
    assert (a - b).abs().max().item() < 0.03 * max(1.0, b.abs().max().item())
    q = torch.randn(4, 192 * 4, generator=g).bfloat16().to(dev)
    assert ops.softmax_attention_mfma_ok(q, 192, 128, 4, 1) and ops.softmax_attention_mfma_ok(q, 96, 64, 8, 1)
    assert not ops.softmax_attention_mfma_ok(q, 112, 96, 4, 1)
    # prompt portions of unequal length with earlier context: two heads per wave against one
    Hh, Wk, dv, npg = 6, 192, 128, 40
    page = (0.4 * torch.randn(npg, 1, 64, Wk, generator=g)).bfloat16().to(dev)
    bt = torch.randperm(npg, generator=g).to(torch.int32).view(2, 20).to(dev)
    cu = torch.tensor([0, 301, 370], dtype=torch.int32, device=dev)
    ctx = torch.tensor([1000, 69], dtype=torch.int32, device=dev)
    qq = torch.randn(370, Hh * Wk, generator=g).bfloat16().to(dev)
    outs = []
    for form in (0, 1):
        with ops.kernel_forms(sm_share_heads=form):
            outs.append(ops.softmax_attention_prefill(qq, page, page, bt, cu, ctx, 301, Hh, 1, Wk, dv, scale=0.07,
                                                      v_in_k=True).float())
    seq, pos = ops._rows_of_portions(cu, ctx, 370, dev)
    want = ops.softmax_attention(qq, page, page, bt, seq, pos, Hh, 1, Wk, dv, scale=0.07, v_in_k=True).float()
    for o in outs:
        assert (o - want).abs().max().item() < 0.03 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("device", DEVICES)
def test_trace_runner_replays_a_schedule(device, tmp_path, monkeypatch, capsys):
    """The trace runner on a model folder: steps as JSON lines on standard input (a prompt in two
    portions, a second request beside single tokens of the first, requests ended and their names
    used again), logits files of the wanted places, a ``done`` line per step."""
    import io

    import numpy as np

    from nv_genai_amd.tools import trace_run
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_dict([lat(mlp=moe()), lat2(mlp=dense())])
    cfg = LumepelConfig.from_dict(cd)
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
    close(rows(0), wa[[0, 64]], "float32", "first portion")
    close(rows(2), torch.stack([wb[28], wa[78]]), "float32", "a portion beside a single token")
    close(rows(3), torch.stack([wa[79], wb[29]]), "float32", "last tokens")
    close(rows(4), wb[4:5], "float32", "a name used again")
