"""The layer-list designs (Bidasun, Biruvik, Lumepel, Lizezen) beside the closest Llama-layout model at
equal sizes (Mistral with a sliding window; Mixtral for Lumepel and Lizezen, whose feed-forwards are
routed experts):
prefill and decode throughput through the serving engine, and the design's kernels alone with
their distance from the roofline. Random weights, synthetic token ids.

    python bench.py --workload designs [--design-sizes s,m,l] [--design-models bidasun,biruvik,lumepel,lizezen]

Prints one JSON line (``metric: design_compare``); bench.py's default workload is untouched.
"""
from __future__ import annotations

import json
import time

import torch

SIZES = {
    # name: hidden, heads, kv_heads, head size, ffn, window, layers, prompts x tokens, decode rows x context
    "s": dict(hidden=1024, heads=8, kv=2, d=128, ffn=2816, window=1024, layers=4, pf=(8, 2048), dec=(64, 2048)),
    "m": dict(hidden=2048, heads=16, kv=4, d=128, ffn=5632, window=2048, layers=4, pf=(4, 4096), dec=(64, 4096)),
    "l": dict(hidden=4096, heads=32, kv=8, d=128, ffn=14336, window=4096, layers=2, pf=(2, 8192), dec=(64, 8192)),
}
VOCAB = 32768
PEAK_BF16 = 2.5e15      # dense MFMA flop/s
PEAK_HBM = 8.0e12       # bytes/s
PEAK_TRANS = 256 * 16 * 2.4e9   # transcendental lanes/s: 256 CUs x 4 SIMDs x 4 lanes/clk at 2.4 GHz
PEAK_VALU = 256 * 4 * 16 * 2 * 2.4e9   # fp32 flop/s of the vector ALUs (FMA = 2), unpacked
BIRUVIK_PATTERN = ("attention", "latent_attention", "hgrn2", "attention")
BIRUVIK_RANK = 256    # latent size of the latent-attention layers
# Lumepel: latent + rotated key part per size (key rows of 192 / 320 elements), query latent, experts
LUMEPEL = {"s": dict(rank=128, rot=64, q_rank=384, experts=8, top=2, eff=1024),
           "m": dict(rank=256, rot=64, q_rank=768, experts=16, top=2, eff=1408),
           "l": dict(rank=256, rot=64, q_rank=1536, experts=32, top=4, eff=2048)}
LUMEPEL_PATTERN = ("latent_attention", "latent_attention_2")
# Lizezen: mLSTM heads of 64-wide keys and 128-wide values, rotary GQA attention with and without
# head norms / score cap / head gate; every second feed-forward a mixture (expert sizes of LUMEPEL)
# with two identity experts, four groups of which two are kept, and a shared expert
LIZEZEN_PATTERN = ("mlstm", "attention", "mlstm", "attention_2")
LIZEZEN_MLSTM = dict(dim=64, vdim=128)
BASELINE_OF = {"bidasun": "mistral", "biruvik": "mistral", "lumepel": "mixtral", "lizezen": "mixtral"}


def _engine(kind: str, z: dict, max_len: int, pages: int, seqs: int):
    from nv_genai_amd.engine.llm_engine import EngineConfig, LLMEngine
    from nv_genai_amd.models.config import LlamaConfig, bidasun_uniform, biruvik_layers, lizezen_layers, lumepel_layers

    if kind == "lizezen":
        u = z["lumepel"]
        pat = [LIZEZEN_PATTERN[i % len(LIZEZEN_PATTERN)] for i in range(z["layers"])]
        mcfg = lizezen_layers(pat, z["hidden"], z["heads"], z["kv"], z["d"], z["d"], z["ffn"], mlstm_heads=z["heads"],
                              mlstm_dim=LIZEZEN_MLSTM["dim"], mlstm_vdim=LIZEZEN_MLSTM["vdim"], experts=u["experts"] - 2,
                              top=u["top"], expert_ff=u["eff"], shared_ff=u["eff"], identity=2, groups=4, keep=2,
                              route_scale=2.0, softcap=30.0, rot_base=1e6, yarn=(8.0, 4096, 32.0, 1.0), vocab_size=VOCAB)
    elif kind == "lumepel":
        u = z["lumepel"]
        pat = [LUMEPEL_PATTERN[i % len(LUMEPEL_PATTERN)] for i in range(z["layers"])]
        mcfg = lumepel_layers(pat, z["hidden"], z["heads"], z["d"], u["rot"], z["d"], u["rank"], u["q_rank"], 0,
                              experts=u["experts"], top=u["top"], expert_ff=u["eff"], shared_ff=u["eff"],
                              yarn=(8.0, 4096, 32.0, 1.0), vocab_size=VOCAB)
    elif kind == "mixtral":
        u = z["lumepel"]
        mcfg = LlamaConfig(name="mixtral-eq", arch="mixtral", vocab_size=VOCAB, hidden=z["hidden"], layers=z["layers"],
                           heads=z["heads"], kv_heads=z["kv"], head_dim=z["d"], ffn=u["eff"], num_experts=u["experts"],
                           experts_per_tok=u["top"], max_position=max_len, rope_theta=1e6, eos_ids=(2,), bos_id=1)
    elif kind == "biruvik":
        pat = [BIRUVIK_PATTERN[i % len(BIRUVIK_PATTERN)] for i in range(z["layers"])]
        mcfg = biruvik_layers(pat, z["hidden"], z["heads"], z["kv"], z["d"], z["d"], z["ffn"], window=z["window"],
                              kv_rank=BIRUVIK_RANK, vocab_size=VOCAB)
    elif kind == "bidasun":
        mcfg = bidasun_uniform(z["layers"], z["hidden"], z["heads"], z["kv"], z["d"], z["d"], z["ffn"], z["window"], 4,
                               vocab_size=VOCAB, max_position=max_len)
    else:
        mcfg = LlamaConfig(name="mistral-eq", arch="mistral", vocab_size=VOCAB, hidden=z["hidden"], layers=z["layers"],
                           heads=z["heads"], kv_heads=z["kv"], head_dim=z["d"], ffn=z["ffn"],
                           sliding_window=z["window"], max_position=max_len, rope_theta=1e6, eos_ids=(2,), bos_id=1)
    cfg = EngineConfig(model=mcfg.name, max_num_seqs=seqs, max_batched_tokens=z["pf"][0] * z["pf"][1],
                       max_model_len=max_len, kv_cache_blocks=pages, enable_prefix_caching=False, detokenize=False,
                       use_graphs=True, graph_batch_sizes=(seqs,), mixed_graphs=False, logits_tap=True,
                       tuned_gemms=False, async_decode=False)
    return LLMEngine(cfg, device="cuda", model_cfg=mcfg)


def _timed(fn, n: int) -> float:
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / n


def engine_rates(kind: str, z: dict, steps: int, warmup: int) -> dict:
    """tokens/s of whole-prompt prefill steps and of decode steps (the captured decode graph)."""
    nb, L = z["pf"]
    nd, ctx = z["dec"]
    max_len = max(L, ctx) + 64 * (steps + warmup + 2)
    pages = max(nb * -(-L // 64), nd * -(-(ctx + steps + warmup + 2) // 64)) + 8
    eng = _engine(kind, z, max_len, pages, max(nb, nd))
    g = torch.Generator().manual_seed(0)
    rid = [0]

    def prefill():
        rows = []
        for _ in range(nb):
            rid[0] += 1
            rows.append((rid[0], torch.randint(3, VOCAB, (L,), generator=g).tolist(), [L - 1]))
        eng.replay_step(rows, [r for r, _, _ in rows])

    for _ in range(warmup):
        prefill()
    t_pf = _timed(prefill, steps)
    # decode: nd sequences of ctx tokens (filled in chunks), then single-token steps
    ids = list(range(10_000, 10_000 + nd))
    per = max(1, (nb * L) // ctx)
    for i in range(0, nd, per):
        eng.replay_step([(r, torch.randint(3, VOCAB, (ctx,), generator=g).tolist(), []) for r in ids[i:i + per]], [])

    def decode():
        eng.replay_step([(r, [5], [0]) for r in ids], [])

    for _ in range(warmup):
        decode()
    t_dec = _timed(decode, steps)
    return {"prefill_tok_s": round(nb * L / t_pf), "prefill_ms": round(t_pf * 1e3, 2),
            "decode_tok_s": round(nd / t_dec), "decode_ms": round(t_dec * 1e3, 3),
            "decode_graph": bool(eng.graphs)}


def kernel_times(z: dict, iters: int = 20) -> dict:
    """The attention kernels alone on one layer's shapes: time, and the fraction of the roofline
    (MFMA flops for the prompt kernels, plus the transcendental rate for the sigmoid one, which
    needs a log, an exp and a reciprocal per score; HBM bytes of the visible pages for decode)."""
    from nv_genai_amd import ops

    dev, bf = "cuda", torch.bfloat16
    H, G, D, W = z["heads"], z["kv"], z["d"], z["window"]
    nb, L = z["pf"]
    nd, ctx = z["dec"]
    pages_seq = -(-max(L, ctx) // 64)
    nseq = max(nb, nd)
    npg = nseq * pages_seq
    kc = (torch.randn(npg, G, 64, D, device=dev) * 0.5).to(bf)
    vc = (torch.randn(npg, G, D, 64, device=dev) * 0.5).to(bf)
    bt = torch.arange(npg, dtype=torch.int32, device=dev).view(nseq, pages_seq)
    r1, r2, pb = (torch.full((H,), v, device=dev) for v in (0.7, 0.2, -1.0))
    out = {}
    # ---- prompt portions: nb sequences of L tokens, no earlier context
    T = nb * L
    q = torch.randn(T, H * D, device=dev).to(bf)
    gate = torch.randn(T, H * D, device=dev).to(bf)
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    cx = torch.full((nb,), L, dtype=torch.int32, device=dev)
    pairs = nb * sum(min(i + 1, W) for i in range(L)) * H          # visible (query, key) pairs
    flops = 4.0 * pairs * D
    t_sig = _timed(lambda: ops.sigmoid_attention_prefill(q, gate, kc, vc, bt, cu, cx, L, H, G, D, D, D ** -0.5, W, 4,
                                                         r1, r2, pb), iters)
    t_soft = _timed(lambda: ops.prefill_attention_paged(q, kc, vc, bt, cu, cx, H, G, D, L, D ** -0.5, window=W, impl=4),
                    iters)
    out["prefill"] = {
        "sigmoid_ms": round(t_sig * 1e3, 3), "softmax_ms": round(t_soft * 1e3, 3),
        "sigmoid_mfma_frac": round(flops / t_sig / PEAK_BF16, 4), "softmax_mfma_frac": round(flops / t_soft / PEAK_BF16, 4),
        "sigmoid_transcendental_frac": round(3.0 * pairs / t_sig / PEAK_TRANS, 4),
        "softmax_transcendental_frac": round(1.0 * pairs / t_soft / PEAK_TRANS, 4)}
    # ---- decode rows: nd sequences of ctx keys, one query each
    qd = torch.randn(nd, H * D, device=dev).to(bf)
    gd = torch.randn(nd, H * D, device=dev).to(bf)
    seq = torch.arange(nd, dtype=torch.int32, device=dev)
    pos = torch.full((nd,), ctx - 1, dtype=torch.int32, device=dev)
    cxd = torch.full((nd,), ctx, dtype=torch.int32, device=dev)
    ws = ops.DecodeWorkspace(nd, H, G, ctx, dev, None, D=D)
    vis = min(ctx, W)
    kv_bytes = nd * G * vis * D * 2 * 2.0
    t_sigd = _timed(lambda: ops.sigmoid_attention_rows(qd, gd, kc, vc, bt, seq, pos, H, G, D, D, D ** -0.5, W, 4, r1, r2,
                                                       pb, max_ctx=ctx), iters)
    t_softd = _timed(lambda: ops.decode_attention(qd, kc, vc, bt, cxd, H, G, ctx, D ** -0.5, ws=ws, window=W), iters)
    out["decode"] = {"sigmoid_ms": round(t_sigd * 1e3, 4), "softmax_ms": round(t_softd * 1e3, 4),
                     "sigmoid_hbm_frac": round(kv_bytes / t_sigd / PEAK_HBM, 4),
                     "softmax_hbm_frac": round(kv_bytes / t_softd / PEAK_HBM, 4)}
    return out


def biruvik_kernel_times(z: dict, iters: int = 20) -> dict:
    """The Biruvik mixer kernels alone on one layer's shapes beside the softmax kernels of the
    Llama layout: differential attention (two maps, causal) against causal softmax attention,
    windowed latent attention (multi-query over the latent page) against windowed softmax
    attention, and the HGRN2 scan (no counterpart: priced against the fp32 vector rate for prompts
    and against the HBM bytes of the state for single rows)."""
    from nv_genai_amd import ops

    dev, bf = "cuda", torch.bfloat16
    H, G, D, W, R = z["heads"], z["kv"], z["d"], z["window"], BIRUVIK_RANK
    nb, L = z["pf"]
    nd, ctx = z["dec"]
    pages_seq = -(-max(L, ctx) // 64)
    nseq = max(nb, nd)
    npg = nseq * pages_seq
    bt = torch.arange(npg, dtype=torch.int32, device=dev).view(nseq, pages_seq)
    k2 = (torch.randn(npg, 2 * G, 64, D, device=dev) * 0.5).to(bf)      # both maps
    vr = (torch.randn(npg, G, 64, D, device=dev) * 0.5).to(bf)          # row-major values
    cc = (torch.randn(npg, 1, 64, R, device=dev) * 0.5).to(bf)          # latent pages
    kl = k2[:, :G].contiguous()
    vt = vr.transpose(2, 3).contiguous()                               # V^T pages of the Llama layout
    T = nb * L
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    cx = torch.full((nb,), L, dtype=torch.int32, device=dev)
    out = {}
    # ---- prompt portions
    q2 = torch.randn(T, H * 2 * D, device=dev).to(bf)
    q1 = q2[:, :H * D].contiguous()
    ql = torch.randn(T, H * R, device=dev).to(bf)
    gate = torch.randn(T, H, device=dev).to(bf)
    pairs_c = nb * (L * (L + 1) // 2) * H
    pairs_w = nb * sum(min(i + 1, W) for i in range(L)) * H
    t_diff = _timed(lambda: ops.softmax_attention_prefill(q2, k2, vr, bt, cu, cx, L, H, G, D, D, D ** -0.5, maps=2,
                                                          lam=0.4, unit_eps=1e-5, out_scale=0.7), iters)
    t_soft_c = _timed(lambda: ops.prefill_attention_paged(q1, kl, vt, bt, cu, cx, H, G, D, L, D ** -0.5, window=0, impl=4),
                      iters)
    t_lat = _timed(lambda: ops.softmax_attention_prefill(ql, cc, cc, bt, cu, cx, L, H, 1, R, R, D ** -0.5, window=W,
                                                         gate=gate), iters)
    t_soft_w = _timed(lambda: ops.prefill_attention_paged(q1, kl, vt, bt, cu, cx, H, G, D, L, D ** -0.5, window=W, impl=4),
                      iters)
    out["prefill"] = {
        "differential_ms": round(t_diff * 1e3, 3), "softmax_causal_ms": round(t_soft_c * 1e3, 3),
        "differential_mfma_frac": round(2 * 4.0 * pairs_c * D / t_diff / PEAK_BF16, 4),
        "softmax_causal_mfma_frac": round(4.0 * pairs_c * D / t_soft_c / PEAK_BF16, 4),
        "latent_ms": round(t_lat * 1e3, 3), "softmax_window_ms": round(t_soft_w * 1e3, 3),
        "latent_mfma_frac": round(4.0 * pairs_w * R / t_lat / PEAK_BF16, 4),
        "softmax_window_mfma_frac": round(4.0 * pairs_w * D / t_soft_w / PEAK_BF16, 4)}
    # ---- single-token rows
    seq = torch.arange(nd, dtype=torch.int32, device=dev)
    pos = torch.full((nd,), ctx - 1, dtype=torch.int32, device=dev)
    cxd = torch.full((nd,), ctx, dtype=torch.int32, device=dev)
    ws = ops.DecodeWorkspace(nd, H, G, ctx, dev, None, D=D)
    t_diffd = _timed(lambda: ops.softmax_attention_rows(q2[:nd], k2, vr, bt, seq, pos, H, G, D, D, D ** -0.5, max_ctx=ctx,
                                                        maps=2, lam=0.4, unit_eps=1e-5, out_scale=0.7), iters)
    t_softd_c = _timed(lambda: ops.decode_attention(q1[:nd], kl, vt, bt, cxd, H, G, ctx, D ** -0.5, ws=ws, window=0), iters)
    t_latd = _timed(lambda: ops.softmax_attention_rows(ql[:nd], cc, cc, bt, seq, pos, H, 1, R, R, D ** -0.5, max_ctx=ctx,
                                                       window=W, gate=gate[:nd]), iters)
    t_softd_w = _timed(lambda: ops.decode_attention(q1[:nd], kl, vt, bt, cxd, H, G, ctx, D ** -0.5, ws=ws, window=W), iters)
    vis = min(ctx, W)
    out["decode"] = {
        "differential_ms": round(t_diffd * 1e3, 4), "softmax_causal_ms": round(t_softd_c * 1e3, 4),
        "differential_hbm_frac": round(nd * G * ctx * 3 * D * 2.0 / t_diffd / PEAK_HBM, 4),
        "softmax_causal_hbm_frac": round(nd * G * ctx * 2 * D * 2.0 / t_softd_c / PEAK_HBM, 4),
        "latent_ms": round(t_latd * 1e3, 4), "softmax_window_ms": round(t_softd_w * 1e3, 4),
        "latent_hbm_frac": round(nd * vis * R * 2.0 / t_latd / PEAK_HBM, 4),
        "softmax_window_hbm_frac": round(nd * G * vis * 2 * D * 2.0 / t_softd_w / PEAK_HBM, 4)}
    # ---- HGRN2 scan: prompts of L rows, then one row per sequence
    proj = torch.randn(T, 3 * H * D, device=dev).to(bf)
    fb = torch.zeros(H * D, device=dev)
    low = torch.full((H * D,), 0.3, device=dev)
    state = torch.zeros(nseq, H, D, D, device=dev)
    slots_p = torch.arange(nb, dtype=torch.int32, device=dev)
    pos_p = torch.arange(L, dtype=torch.int32, device=dev).repeat(nb)
    t_scan = _timed(lambda: ops.hgrn2_scan(proj, fb, low, state, H, D, D, cu, slots_p, pos_p), max(2, iters // 4))
    t_scand = _timed(lambda: ops.hgrn2_scan(proj[:nd], fb, low, state, H, D, D, None, seq, pos), iters)
    out["hgrn2"] = {"prefill_ms": round(t_scan * 1e3, 3), "prefill_tok_s": round(T / t_scan),
                    "prefill_valu_frac": round(6.0 * T * H * D * D / t_scan / PEAK_VALU, 4),
                    "decode_ms": round(t_scand * 1e3, 4),
                    "decode_hbm_frac": round(nd * H * D * D * 4 * 2.0 / t_scand / PEAK_HBM, 4)}
    return out


def lumepel_kernel_times(z: dict, iters: int = 20) -> dict:
    """The Lumepel kernels alone on one layer's shapes beside the like kernels of the Llama layout:
    latent attention (multi-query over the page of [latent | rotated key part] rows, values inside
    the key rows) against causal softmax attention, the routed clamped-GLU experts against the
    Mixtral experts, and the row kernels (latent norm + rotation + page write against rotation +
    KV write; residual sum + norm; gated activation) against their counterparts, priced by the
    bytes they must move."""
    from nv_genai_amd import ops
    from nv_genai_amd.ops import reference as ref

    dev, bf = "cuda", torch.bfloat16
    u = z["lumepel"]
    H, G, D, R, RD = z["heads"], z["kv"], z["d"], u["rank"], u["rot"]
    Wk = R + RD
    nb, L = z["pf"]
    nd, ctx = z["dec"]
    pages_seq = -(-max(L, ctx) // 64)
    nseq = max(nb, nd)
    npg = nseq * pages_seq
    bt = torch.arange(npg, dtype=torch.int32, device=dev).view(nseq, pages_seq)
    page = (torch.randn(npg, 1, 64, Wk, device=dev) * 0.5).to(bf)
    kl = (torch.randn(npg, G, 64, D, device=dev) * 0.5).to(bf)
    vt = (torch.randn(npg, G, D, 64, device=dev) * 0.5).to(bf)
    T = nb * L
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    cx = torch.full((nb,), L, dtype=torch.int32, device=dev)
    ql = torch.randn(T, H * Wk, device=dev).to(bf)
    q1 = torch.randn(T, H * D, device=dev).to(bf)
    pairs = nb * (L * (L + 1) // 2) * H
    sc = (D + RD) ** -0.5
    out = {"mfma_attention": bool(ops.softmax_attention_mfma_ok(ql, Wk, R, H, 1))}
    t_lat = _timed(lambda: ops.softmax_attention_prefill(ql, page, page, bt, cu, cx, L, H, 1, Wk, R, sc, v_in_k=True), iters)
    t_soft = _timed(lambda: ops.prefill_attention_paged(q1, kl, vt, bt, cu, cx, H, G, D, L, D ** -0.5, window=0, impl=4),
                    iters)
    out["prefill"] = {"latent_ms": round(t_lat * 1e3, 3), "softmax_ms": round(t_soft * 1e3, 3),
                      "latent_mfma_frac": round(2.0 * pairs * (Wk + R) / t_lat / PEAK_BF16, 4),
                      "softmax_mfma_frac": round(4.0 * pairs * D / t_soft / PEAK_BF16, 4)}
    seq = torch.arange(nd, dtype=torch.int32, device=dev)
    pos = torch.full((nd,), ctx - 1, dtype=torch.int32, device=dev)
    cxd = torch.full((nd,), ctx, dtype=torch.int32, device=dev)
    ws = ops.DecodeWorkspace(nd, H, G, ctx, dev, None, D=D)
    t_latd = _timed(lambda: ops.softmax_attention_rows(ql[:nd], page, page, bt, seq, pos, H, 1, Wk, R, sc, max_ctx=ctx,
                                                       v_in_k=True), iters)
    t_softd = _timed(lambda: ops.decode_attention(q1[:nd], kl, vt, bt, cxd, H, G, ctx, D ** -0.5, ws=ws, window=0), iters)
    out["decode"] = {"latent_ms": round(t_latd * 1e3, 4), "softmax_ms": round(t_softd * 1e3, 4),
                     "latent_hbm_frac": round(nd * ctx * Wk * 2.0 / t_latd / PEAK_HBM, 4),
                     "softmax_hbm_frac": round(nd * G * ctx * 2 * D * 2.0 / t_softd / PEAK_HBM, 4)}
    # ---- experts: T rows (prompts) and nd rows (single tokens)
    Hd, E, k, F = z["hidden"], u["experts"], u["top"], u["eff"]
    x = torch.randn(T, Hd, device=dev).to(bf)
    router = (torch.randn(E, Hd, device=dev) * Hd ** -0.5)
    w13 = (torch.randn(E, 2 * F, Hd, device=dev) * Hd ** -0.5).to(bf)
    w2 = (torch.randn(E, Hd, F, device=dev) * F ** -0.5).to(bf)
    rb = router.to(bf)

    def lum(xx):
        ids, wts = ops.moe_route_scores(ops.linear(xx.float(), router), k, "sigmoid", False)
        return ops.moe_glu_experts(xx, ids, wts, w13, w2, 7.0, 1.702, True)

    ex = {}
    for name, rows in (("prefill", T), ("decode", nd)):
        xx = x[:rows]
        fl = 2.0 * rows * k * 3 * Hd * F
        by = min(E, rows * k) * 3 * Hd * F * 2.0
        t_l = _timed(lambda: lum(xx), iters)
        t_m = _timed(lambda: ops.moe_ffn(xx, rb, w13, w2, k), iters)
        ex[name] = {"lumepel_ms": round(t_l * 1e3, 3), "mixtral_ms": round(t_m * 1e3, 3),
                    "lumepel_mfma_frac": round(fl / t_l / PEAK_BF16, 4), "mixtral_mfma_frac": round(fl / t_m / PEAK_BF16, 4),
                    "lumepel_weight_hbm_frac": round(by / t_l / PEAK_HBM, 4),
                    "mixtral_weight_hbm_frac": round(by / t_m / PEAK_HBM, 4)}
    out["experts"] = ex
    del x, w13, w2
    # ---- row kernels (prompt rows): bytes that must move over the time, against 8 TB/s
    nq = H * (D + RD)
    proj = torch.randn(T, nq + Wk, device=dev).to(bf)
    qf = torch.empty(T, H * Wk, device=dev, dtype=bf)
    posr = torch.arange(L, dtype=torch.int32, device=dev).repeat(nb)
    slots = torch.arange(T, dtype=torch.int32, device=dev)
    freq, mag = ops.rotary_frequencies(RD, 1e4, (8.0, 4096, 32.0, 1.0))
    freq = freq.to(dev)
    cw = torch.ones(R, device=dev)
    t_rc = _timed(lambda: ops.latent_rope_cache_(proj, posr, slots, page, freq, mag, True, RD, RD, 1e-5, kv=(nq, R, cw),
                                                 q=(0, H, D), q_out=qf), iters)
    by_rc = T * (2 * H * RD + 2 * Wk) * 2.0              # rotated parts read + written, latent row read + written
    qkv = torch.randn(T, (H + 2 * G) * D, device=dev).to(bf)
    cs = ref.rope_cos_sin(L, D, 1e6).to(dev)
    t_rk = _timed(lambda: ops.rope_cache_(qkv, posr, cs, slots, kl, vt, H, G, D), iters)
    by_rk = T * (2 * (H + G) * D + 2 * G * D) * 2.0      # q, k read + written, k and v pages written, v read
    xs = torch.randn(T, Hd, device=dev)
    y = torch.randn(T, Hd, device=dev).to(bf)
    wn = torch.ones(Hd, device=dev)
    t_rn = _timed(lambda: ops.residual_add_rmsnorm_(xs, y, wn, 1e-5, bf), iters)
    xb = xs.to(bf)
    wb = wn.to(bf)
    t_an = _timed(lambda: ops.add_rmsnorm(xb, y, wb, 1e-5), iters)
    Fd = 4 * Hd
    gu = torch.randn(T, 2 * Fd, device=dev).to(bf)
    t_cg = _timed(lambda: ops.clamped_glu(gu, Fd, 7.0), iters)
    t_sm = _timed(lambda: ops.silu_mul(gu), iters)
    out["rows"] = {
        "latent_rope_cache_ms": round(t_rc * 1e3, 3), "latent_rope_cache_hbm_frac": round(by_rc / t_rc / PEAK_HBM, 4),
        "rope_cache_ms": round(t_rk * 1e3, 3), "rope_cache_hbm_frac": round(by_rk / t_rk / PEAK_HBM, 4),
        "residual_add_rmsnorm_ms": round(t_rn * 1e3, 3),
        "residual_add_rmsnorm_hbm_frac": round(T * Hd * 12.0 / t_rn / PEAK_HBM, 4),     # fp32 in + out, bf16 in + out
        "add_rmsnorm_ms": round(t_an * 1e3, 3), "add_rmsnorm_hbm_frac": round(T * Hd * 8.0 / t_an / PEAK_HBM, 4),
        "clamped_glu_ms": round(t_cg * 1e3, 3), "clamped_glu_hbm_frac": round(T * Fd * 6.0 / t_cg / PEAK_HBM, 4),
        "silu_mul_ms": round(t_sm * 1e3, 3), "silu_mul_hbm_frac": round(T * Fd * 6.0 / t_sm / PEAK_HBM, 4)}
    return out


def lizezen_kernel_times(z: dict, iters: int = 20) -> dict:
    """The Lizezen kernels alone on one layer's shapes beside the like kernels of the other models:
    the mLSTM scan against the HGRN2 scan (same state size), rotary GQA attention with head gate
    and capped scores against causal softmax attention of the Llama layout, the group-routed SwiGLU
    experts with identity experts against the Mixtral experts, and the row kernels (head norms +
    rotation + page write against rotation + KV write; parallel residual step with the dynamic tanh
    against residual sum + RMS norm; GELU with bias against the gated activation), priced by the
    flops or bytes they must move."""
    from nv_genai_amd import ops
    from nv_genai_amd.ops import reference as ref

    dev, bf = "cuda", torch.bfloat16
    u = z["lumepel"]
    H, G, D = z["heads"], z["kv"], z["d"]
    d, dv = LIZEZEN_MLSTM["dim"], LIZEZEN_MLSTM["vdim"]
    nb, L = z["pf"]
    nd, ctx = z["dec"]
    T = nb * L
    out = {}
    # ---- scans: prompts (nb segments of L rows) and single rows (nd segments)
    nq, nv = H * d, H * dv
    proj = torch.randn(T, 2 * nq + 2 * nv + 2 * H, device=dev).to(bf)
    gb = torch.randn(2 * H, device=dev)
    st = torch.zeros(max(nb, nd), H, ops.mlstm_state_size(d, dv), device=dev)
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    posr = torch.arange(L, dtype=torch.int32, device=dev).repeat(nb)
    sl_p = torch.arange(nb, dtype=torch.int32, device=dev)
    sl_d = torch.arange(nd, dtype=torch.int32, device=dev)
    posd = torch.full((nd,), ctx - 1, dtype=torch.int32, device=dev)
    offs = (0, nq, 2 * nq, 2 * nq + 2 * nv)
    t_mp = _timed(lambda: ops.mlstm_scan(proj, gb, st, H, d, dv, 15.0, cu, sl_p, posr, offs), iters)
    t_md = _timed(lambda: ops.mlstm_scan(proj[:nd], gb, st, H, d, dv, 15.0, None, sl_d, posd, offs), iters)
    hp = torch.randn(T, 2 * nq + nv, device=dev).to(bf)
    fb, lw = torch.randn(nq, device=dev), torch.rand(nq, device=dev) * 0.9
    hs = torch.zeros(max(nb, nd), H, d, dv, device=dev)
    t_hp = _timed(lambda: ops.hgrn2_scan(hp, fb, lw, hs, H, d, dv, cu, sl_p, posr), iters)
    t_hd = _timed(lambda: ops.hgrn2_scan(hp[:nd], fb, lw, hs, H, d, dv, None, sl_d, posd), iters)
    fl = 6.0 * T * H * d * dv                              # 3 FMAs per state element and row
    by = nd * H * d * dv * 8.0                             # state read + written
    out["scan"] = {"mlstm_prefill_ms": round(t_mp * 1e3, 3), "hgrn2_prefill_ms": round(t_hp * 1e3, 3),
                   "mlstm_valu_frac": round(fl / t_mp / PEAK_VALU, 4), "hgrn2_valu_frac": round(fl / t_hp / PEAK_VALU, 4),
                   "mlstm_decode_ms": round(t_md * 1e3, 4), "hgrn2_decode_ms": round(t_hd * 1e3, 4),
                   "mlstm_state_hbm_frac": round(by / t_md / PEAK_HBM, 4), "hgrn2_state_hbm_frac": round(by / t_hd / PEAK_HBM, 4)}
    del proj, hp
    # ---- attention: capped scores and a head gate on row-major pages against the Llama-layout kernels
    pages_seq = -(-max(L, ctx) // 64)
    nseq = max(nb, nd)
    npg = nseq * pages_seq
    bt = torch.arange(npg, dtype=torch.int32, device=dev).view(nseq, pages_seq)
    kr = (torch.randn(npg, G, 64, D, device=dev) * 0.5).to(bf)
    vr = (torch.randn(npg, G, 64, D, device=dev) * 0.5).to(bf)
    vt = (torch.randn(npg, G, D, 64, device=dev) * 0.5).to(bf)
    cx = torch.full((nb,), L, dtype=torch.int32, device=dev)
    q1 = torch.randn(T, H * D, device=dev).to(bf)
    gate = torch.randn(T, H, device=dev).to(bf)
    pairs = nb * (L * (L + 1) // 2) * H
    sc = D ** -0.5
    out["mfma_attention"] = bool(ops.softmax_attention_mfma_ok(q1, D, D, H // G, 1))
    t_cap = _timed(lambda: ops.softmax_attention_prefill(q1, kr, vr, bt, cu, cx, L, H, G, D, D, sc, softcap=30.0, gate=gate),
                   iters)
    t_pl = _timed(lambda: ops.softmax_attention_prefill(q1, kr, vr, bt, cu, cx, L, H, G, D, D, sc), iters)
    t_soft = _timed(lambda: ops.prefill_attention_paged(q1, kr, vt, bt, cu, cx, H, G, D, L, sc, window=0, impl=4), iters)
    out["prefill"] = {"capped_gated_ms": round(t_cap * 1e3, 3), "plain_ms": round(t_pl * 1e3, 3),
                      "llama_layout_ms": round(t_soft * 1e3, 3),
                      "capped_gated_mfma_frac": round(4.0 * pairs * D / t_cap / PEAK_BF16, 4),
                      "plain_mfma_frac": round(4.0 * pairs * D / t_pl / PEAK_BF16, 4),
                      "llama_layout_mfma_frac": round(4.0 * pairs * D / t_soft / PEAK_BF16, 4)}
    seq = torch.arange(nd, dtype=torch.int32, device=dev)
    cxd = torch.full((nd,), ctx, dtype=torch.int32, device=dev)
    ws = ops.DecodeWorkspace(nd, H, G, ctx, dev, None, D=D)
    t_capd = _timed(lambda: ops.softmax_attention_rows(q1[:nd], kr, vr, bt, seq, posd, H, G, D, D, sc, max_ctx=ctx,
                                                       softcap=30.0, gate=gate[:nd]), iters)
    t_softd = _timed(lambda: ops.decode_attention(q1[:nd], kr, vt, bt, cxd, H, G, ctx, sc, ws=ws, window=0), iters)
    kvb = nd * G * ctx * 2 * D * 2.0
    out["decode"] = {"capped_gated_ms": round(t_capd * 1e3, 4), "llama_layout_ms": round(t_softd * 1e3, 4),
                     "capped_gated_hbm_frac": round(kvb / t_capd / PEAK_HBM, 4),
                     "llama_layout_hbm_frac": round(kvb / t_softd / PEAK_HBM, 4)}
    # ---- experts: T rows (prompts) and nd rows (single tokens)
    Hd, E, k, F = z["hidden"], u["experts"], u["top"], u["eff"]
    x = torch.randn(T, Hd, device=dev).to(bf)
    router = (torch.randn(E, Hd, device=dev) * Hd ** -0.5)
    corr = torch.randn(E, device=dev) * 0.5 / E
    w13 = (torch.randn(E, 2 * F, Hd, device=dev) * Hd ** -0.5).to(bf)
    w2 = (torch.randn(E, Hd, F, device=dev) * F ** -0.5).to(bf)
    rb = router.to(bf)

    def liz(xx):     # the last two router outputs are identity experts
        ids, wts = ops.moe_route_grouped(ops.linear(xx.float(), router), corr, k, 4, 2, 2.0)
        return ops.moe_glu_experts(xx, ids, wts, w13[:E - 2], w2[:E - 2], float("inf"), 1.0, False, shift=0.0, identity=True)

    ex = {}
    for name, rows in (("prefill", T), ("decode", nd)):
        xx = x[:rows]
        fl = 2.0 * rows * k * 3 * Hd * F
        by = min(E, rows * k) * 3 * Hd * F * 2.0
        t_l = _timed(lambda: liz(xx), iters)
        t_m = _timed(lambda: ops.moe_ffn(xx, rb, w13, w2, k), iters)
        ex[name] = {"lizezen_ms": round(t_l * 1e3, 3), "mixtral_ms": round(t_m * 1e3, 3),
                    "lizezen_mfma_frac": round(fl / t_l / PEAK_BF16, 4), "mixtral_mfma_frac": round(fl / t_m / PEAK_BF16, 4),
                    "lizezen_weight_hbm_frac": round(by / t_l / PEAK_HBM, 4),
                    "mixtral_weight_hbm_frac": round(by / t_m / PEAK_HBM, 4)}
    out["experts"] = ex
    del x, w13, w2
    # ---- row kernels (prompt rows): bytes that must move over the time, against 8 TB/s
    qkv = torch.randn(T, (H + 2 * G) * D, device=dev).to(bf)
    slots = torch.arange(T, dtype=torch.int32, device=dev)
    freq, mag = ops.rotary_frequencies(D, 1e6, (8.0, 4096, 32.0, 1.0))
    freq = freq.to(dev)
    hw = torch.ones(D, device=dev)
    t_rh = _timed(lambda: ops.rope_headnorm_cache_(qkv, posr, slots, kr, vr, H, G, D, D, freq, mag, D, 1e-5, q_w=hw, k_w=hw,
                                                   v_off=(H + G) * D), iters)
    cs = ref.rope_cos_sin(L, D, 1e6).to(dev)
    t_rk = _timed(lambda: ops.rope_cache_(qkv, posr, cs, slots, kr, vt, H, G, D), iters)
    by_rk = T * (2 * (H + G) * D + 2 * G * D) * 2.0      # q, k read + written, k and v pages written, v read
    xs = torch.randn(T, Hd, device=dev)
    y1, y2 = torch.randn(T, Hd, device=dev).to(bf), torch.randn(T, Hd, device=dev).to(bf)
    wn, bn = torch.ones(Hd, device=dev), torch.zeros(Hd, device=dev)
    t_rd = _timed(lambda: ops.residual_dyt_(xs, y1, y2, bn, (0.5, wn, bn), bf), iters)
    xb, wb = xs.to(bf), wn.to(bf)
    t_an = _timed(lambda: ops.add_rmsnorm(xb, y1, wb, 1e-5), iters)
    Fd = z["ffn"] // 8 * 8
    up = torch.randn(T, Fd, device=dev).to(bf)
    gu = torch.randn(T, 2 * Fd, device=dev).to(bf)
    bu = torch.randn(Fd, device=dev)
    t_bg = _timed(lambda: ops.bias_gelu_tanh_(up, bu), iters)
    t_sm = _timed(lambda: ops.silu_mul(gu), iters)
    o = torch.randn(T, nv, device=dev)
    gg = torch.randn(T, nv, device=dev).to(bf)
    won = torch.ones(nv, device=dev)
    t_gn = _timed(lambda: ops.group_rmsnorm(o, won, H, 1e-5, bf, gate=gg), iters)
    out["rows"] = {
        "rope_headnorm_cache_ms": round(t_rh * 1e3, 3), "rope_headnorm_cache_hbm_frac": round(by_rk / t_rh / PEAK_HBM, 4),
        "rope_cache_ms": round(t_rk * 1e3, 3), "rope_cache_hbm_frac": round(by_rk / t_rk / PEAK_HBM, 4),
        "residual_dyt_ms": round(t_rd * 1e3, 3),
        "residual_dyt_hbm_frac": round(T * Hd * 14.0 / t_rd / PEAK_HBM, 4),      # fp32 in + out, two bf16 in, bf16 out
        "add_rmsnorm_ms": round(t_an * 1e3, 3), "add_rmsnorm_hbm_frac": round(T * Hd * 8.0 / t_an / PEAK_HBM, 4),
        "bias_gelu_tanh_ms": round(t_bg * 1e3, 3), "bias_gelu_tanh_hbm_frac": round(T * Fd * 4.0 / t_bg / PEAK_HBM, 4),
        "silu_mul_ms": round(t_sm * 1e3, 3), "silu_mul_hbm_frac": round(T * Fd * 6.0 / t_sm / PEAK_HBM, 4),
        "gated_head_norm_ms": round(t_gn * 1e3, 3), "gated_head_norm_hbm_frac": round(T * nv * 8.0 / t_gn / PEAK_HBM, 4)}
    return out


def run(args) -> None:
    names = [s for s in (args.design_sizes or "s,m,l").split(",") if s]
    models = [m for m in (getattr(args, "design_models", None) or "bidasun").split(",") if m]
    if any(m not in BASELINE_OF for m in models):
        raise SystemExit(f"--design-models: unknown design in {models} ({', '.join(BASELINE_OF)})")
    res = {}
    for n in names:
        z = dict(SIZES[n], lumepel=LUMEPEL[n])
        res[n] = {"shape": {k: v for k, v in z.items()}}
        for kind in models + sorted({BASELINE_OF[m] for m in models}):
            res[n][kind] = engine_rates(kind, z, max(1, args.steps), max(1, args.warmup))
            torch.cuda.empty_cache()
        if "bidasun" in models:
            res[n]["attention_kernels"] = kernel_times(z)
            torch.cuda.empty_cache()
        if "biruvik" in models:
            res[n]["biruvik_kernels"] = biruvik_kernel_times(z)
            torch.cuda.empty_cache()
        if "lumepel" in models:
            res[n]["lumepel_kernels"] = lumepel_kernel_times(z)
            torch.cuda.empty_cache()
        if "lizezen" in models:
            res[n]["lizezen_kernels"] = lizezen_kernel_times(z)
            torch.cuda.empty_cache()
        print(f"[designs] {n}: {json.dumps(res[n])}", flush=True)
    line = {"metric": "design_compare", "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "dtype": "bf16", "data": "synthetic token ids, random weights", "sizes": res}
    print(json.dumps(line), flush=True)
    if args.out:
        with open(args.out, "w") as f:
            f.write(json.dumps(line) + "\n")
