"""Nositar (sigmoid head-mixing attention + gated delta rule over fp32 residual streams) against the slow oracle of
tests/nositar_oracle.py: every mechanism alone, then whole models through the engine's own scheduler, page pool, state
slots and step function -- on the CPU backend (fp32) and, marked gpu, through the HIP kernels (fp32 and bf16).
Small random models are written to disk as checkpoints, so the loader and the configuration reader run too."""
import pytest
import torch

import nositar_oracle as O
from vllm_distributed_amd import ops

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 0.12}


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(0)


def hybrid_layers():
    return [O.attention_layer(), O.delta_layer(), O.attention_layer(heads=2, kv_heads=2, dim=8, vdim=24, window=7,
                                                                    keep_first=3),
            O.delta_layer(heads=4, kv_heads=2, dim=12, vdim=16, conv=3, kind="channel_delta_2")]


# ---- driving the engine ------------------------------------------------------------------------------------------
def run_schedule(folder, dtype, device, prompts, schedule, max_tokens, block_size=16, eager=True):
    """``schedule``: steps of (request, token count); every request ends when its tokens are used up.  Returns
    request -> logits [tokens, vocab] in the order the tokens ran."""
    from vllm_distributed_amd.entrypoints.trace_replay import TraceReplayer
    r = TraceReplayer(folder, dtype, max_tokens, block_size=block_size, device=device, enforce_eager=eager)
    at = {k: 0 for k in prompts}
    got = {k: [] for k in prompts}
    try:
        for step in schedule:
            entries, end = [], []
            for rid, n in step:
                lo, hi = at[rid], at[rid] + n
                entries.append({"id": rid, "tokens": prompts[rid][lo:hi], "want": list(range(n))})
                at[rid] = hi
                if hi == len(prompts[rid]):
                    end.append(rid)
            rows = torch.from_numpy(r.step(entries, end))
            o = 0
            for rid, n in step:
                got[rid].append(rows[o:o + n])
                o += n
    finally:
        r.shutdown()
    assert all(at[k] == len(prompts[k]) for k in prompts)
    return {k: torch.cat(v) for k, v in got.items()}


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def check(cfg, W, prompts, got, dtype):
    for rid, p in prompts.items():
        want = O.forward(cfg, W, p)
        err = O.logit_error(got[rid], want)
        assert err < TOL[dtype], f"request {rid}: logits differ by {err:.2e} of their spread"


def model(tmp_path, layers, seed=0, sharp=False, **kw):
    cfg = O.make_config(layers, **kw)
    W = O.make_weights(cfg, seed)
    if sharp:
        # few keys carry almost all of a query's weight: one key too many or too few moves the output by O(1)
        for k in list(W):
            if k.endswith(("mix.q", "mix.k")) and f"{k}.conv" not in W and k.replace("mix.q", "mix.talk").replace(
                    "mix.k", "mix.talk") in W:
                W[k] = (W[k].float() * 2.0).to(W[k].dtype)
            if k.endswith("mix.pb"):
                W[k] = (W[k].float() - 2.5).to(W[k].dtype)
    return O.save_checkpoint(str(tmp_path / "m"), cfg, W), cfg, W


# ---- mechanisms alone ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("n", [1, 2, 3])
def test_streams_read_write(dev, n):
    T, Wd = 5, 40
    xs = torch.randn(n, T, Wd)
    y = torch.randn(T, Wd)
    mix, w_in, w_out = torch.eye(n) + 0.2 * torch.randn(n, n), torch.randn(n), torch.randn(n)
    gain, eps = torch.tensor([1.3]), 1e-5
    new = [sum(mix[s, t] * xs[s] for s in range(n)) + w_out[t] * y for t in range(n)]
    u = sum(w_in[s] * new[s] for s in range(n))
    want_h = O.scalar_norm(u, gain, eps)
    xd = xs.clone().to(dev)
    h = ops.stream_step(xd, y.to(dev), mix.to(dev), w_out.to(dev), w_in=w_in.to(dev), gain=gain.to(dev), eps=eps,
                        out_dtype=torch.float32)
    torch.testing.assert_close(xd.cpu(), torch.stack(new), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(h.cpu(), want_h, atol=1e-5, rtol=1e-5)
    emb = torch.randn(11, Wd)
    ids = torch.tensor([3, 3, 10, 0], dtype=torch.int32)
    e = ops.stream_embed(ids.to(dev), emb.to(dev), 2.5, n)
    torch.testing.assert_close(e.cpu(), (emb[ids.long()] * 2.5).expand(n, -1, -1))


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("H,G,D,E,window,keep", [(4, 2, 16, 16, 9, 2), (3, 3, 20, 8, 5, 0), (8, 4, 40, 24, 40, 3),
                                                 (2, 1, 8, 8, None, 0), (6, 2, 24, 24, 1, 1)])
def test_sigmoid_attention_paged(dev, H, G, D, E, window, keep):
    """Ragged batch on scattered pages -- a decode-form sequence, a portion of a prompt behind cached context, a
    whole prompt -- against the dense oracle of each sequence."""
    bs, eps, scale = 4, 1e-5, 0.3
    lens, news = [23, 37, 14], [1, 9, 14]
    C = H * D + G * D + G * E
    seqs = [torch.randn(n, C) for n in lens]
    talk, pb = torch.eye(H) + 0.4 * torch.randn(H, H), torch.randn(H) - 1.0
    nblk = sum(-(-n // bs) for n in lens) + 3
    perm = torch.randperm(nblk - 1) + 1
    kc = torch.zeros(nblk, G, bs, D, device=dev)
    vc = torch.zeros(nblk, G, E, bs, device=dev)
    table = torch.zeros(len(lens), max(-(-n // bs) for n in lens), dtype=torch.int32)
    o = 0
    for s, n in enumerate(lens):
        k = -(-n // bs)
        table[s, :k] = perm[o:o + k].int()
        o += k
    # context first (as earlier steps would have), then the step's own tokens
    for s, (n, m) in enumerate(zip(lens, news)):
        if n - m:
            slots = torch.tensor([int(table[s, p // bs]) * bs + p % bs for p in range(n - m)])
            ops.unit_rms_qk_and_cache(seqs[s][: n - m].to(dev), H, G, D, E, eps, kc, vc, slots.to(dev))
    x = torch.cat([seqs[s][n - m:] for s, (n, m) in enumerate(zip(lens, news))])
    slots = torch.tensor([int(table[s, p // bs]) * bs + p % bs for s, (n, m) in enumerate(zip(lens, news))
                          for p in range(n - m, n)])
    qn = ops.unit_rms_qk_and_cache(x.to(dev), H, G, D, E, eps, kc, vc, slots.to(dev))
    qsl = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32)
    out = ops.sigmoid_window_attention(qn, kc, vc, table.to(dev), torch.tensor(lens, dtype=torch.int32).to(dev),
                                       qsl.to(dev), talk.to(dev), pb.to(dev), scale, window or 0, keep, max(news),
                                       torch.float32).cpu()
    eye = torch.eye(C)
    o = 0
    for s, (n, m) in enumerate(zip(lens, news)):
        want = O.sigmoid_attention(seqs[s], eye[: H * D], eye[H * D: (H + G) * D], eye[(H + G) * D:],
                                   torch.eye(H * E), talk, pb, H, G, D, E, scale, window, keep, eps)[n - m:]
        torch.testing.assert_close(out[o:o + m], want, atol=2e-5, rtol=2e-5)
        o += m


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,E,window,keep,bs", [(8, 2, 40, 56, 70, 5, 16), (16, 4, 64, 64, 40, 3, 16),
                                                    (4, 4, 128, 128, None, 0, 32), (16, 16, 32, 104, 300, 2, 16),
                                                    (3, 1, 24, 8, 33, 40, 8)])
def test_sigmoid_attention_matrix_core_form(monkeypatch, H, G, D, E, window, keep, bs):
    """The 16-bit form (q.k and weights.v on the matrix cores) against the dense oracle fed with the same bf16
    numbers, and against the plain fp32-arithmetic form of the same kernel family."""
    from vllm_distributed_amd import envs
    eps, scale = 1e-5, D ** -0.5
    lens, news = [150, 333, 40, 129], [1, 70, 40, 17]
    C = H * D + G * D + G * E
    seqs = [torch.randn(n, C).bfloat16() for n in lens]
    talk, pb = torch.eye(H) + 0.3 * torch.randn(H, H), torch.randn(H) - 2.0
    nblk = sum(-(-n // bs) for n in lens) + 2
    perm = torch.randperm(nblk - 1) + 1
    table = torch.zeros(len(lens), max(-(-n // bs) for n in lens), dtype=torch.int32)
    o = 0
    for s, n in enumerate(lens):
        k = -(-n // bs)
        table[s, :k] = perm[o:o + k].int()
        o += k
    outs = {}
    for form in ("mfma", "plain"):
        monkeypatch.setattr(envs, "VDA_SIGMOID_ATTN_FORM", form, raising=False)
        kc = torch.zeros(nblk, G, bs, D, device="cuda", dtype=torch.bfloat16)
        vc = torch.zeros(nblk, G, E, bs, device="cuda", dtype=torch.bfloat16)
        slots = torch.tensor([int(table[s, p // bs]) * bs + p % bs for s, n in enumerate(lens) for p in range(n)])
        qn_all = ops.unit_rms_qk_and_cache(torch.cat(seqs).cuda(), H, G, D, E, eps, kc, vc, slots.cuda())
        starts = torch.tensor([0] + lens).cumsum(0)
        qn = torch.cat([qn_all[starts[s] + n - m: starts[s] + n] for s, (n, m) in enumerate(zip(lens, news))])
        qsl = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32)
        outs[form] = ops.sigmoid_window_attention(qn.contiguous(), kc, vc, table.cuda(),
                                                  torch.tensor(lens, dtype=torch.int32).cuda(), qsl.cuda(), talk.cuda(),
                                                  pb.cuda(), scale, window or 0, keep, max(news), torch.bfloat16
                                                  ).float().cpu()
    eye = torch.eye(C)
    o = 0
    for s, (n, m) in enumerate(zip(lens, news)):
        want = O.sigmoid_attention(seqs[s].float(), eye[: H * D], eye[H * D: (H + G) * D], eye[(H + G) * D:],
                                   torch.eye(H * E), talk, pb, H, G, D, E, scale, window, keep, eps)[n - m:]
        for form in outs:      # weights are not normalised over keys: errors scale with the largest output
            err = (outs[form][o:o + m] - want).abs().max() / want.abs().max()
            assert err < 2e-2, f"{form}: sequence {s} differs by {err:.3f} of the largest output"
        o += m


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("H,G,D,E,taps", [(2, 2, 16, 8, 4), (4, 2, 12, 20, 3), (3, 1, 64, 64, 2), (1, 1, 40, 100, 5)])
def test_delta_rule_carried_state(dev, H, G, D, E, taps):
    """Two sequences run in portions (one of them token by token at the end) in state slots that are not in order,
    against the oracle on the whole sequences."""
    eps, ra, rg = 1e-5, 5, 7
    C = 2 * G * D + H * E
    Wd = C + ra + rg + H
    lens = [21, 9]
    xs = [torch.randn(n, Wd) for n in lens]
    eye = torch.eye(Wd)
    P = {"q": eye[: G * D], "k": eye[G * D: 2 * G * D], "v": eye[2 * G * D: C], "a1": eye[C: C + ra],
         "g1": eye[C + ra: C + ra + rg], "b": eye[C + ra + rg:], "q.conv": 0.6 * torch.randn(G * D, taps),
         "k.conv": 0.6 * torch.randn(G * D, taps), "v.conv": 0.6 * torch.randn(H * E, taps),
         "a2": torch.randn(H * D, ra), "g2": torch.randn(H * E, rg), "A_log": torch.randn(H) * 0.5 - 1,
         "dt_bias": torch.randn(H * D), "norm": 1 + 0.1 * torch.randn(E), "o": torch.eye(H * E)}
    want = [O.delta_rule(x, P, H, G, D, E, eps) for x in xs]
    conv_w = torch.cat([P["q.conv"], P["k.conv"], P["v.conv"]]).to(dev)
    conv_state = torch.full((5, C, taps - 1), 7.0, device=dev)          # stale content of an earlier owner
    state = torch.full((5, H, E, D), 3.0, device=dev)
    slot = torch.tensor([[4], [2]], dtype=torch.int32, device=dev)
    done = [0, 0]
    got = [[], []]
    for step in ([(0, 2), (1, 4)], [(0, 16)], [(1, 1), (0, 1)], [(0, 1), (1, 3)], [(1, 1), (0, 1)]):
        order = sorted(step, key=lambda a: a[1] > 1)                     # one-token sequences first, as the runner does
        x = torch.cat([xs[s][done[s]: done[s] + n] for s, n in order]).to(dev)
        qsl = torch.tensor([0] + list(torch.tensor([n for _, n in order]).cumsum(0)), dtype=torch.int32, device=dev)
        lens_now = torch.tensor([done[s] + n for s, n in order], dtype=torch.int32, device=dev)
        tbl = slot[[s for s, _ in order]]
        xc = ops.causal_conv1d(x[:, :C], conv_w, None, conv_state, qsl, lens_now, tbl, max(n for _, n in order))
        a_raw = x[:, C: C + ra] @ P["a2"].T.to(dev)
        g_raw = x[:, C + ra: C + ra + rg] @ P["g2"].T.to(dev)
        out = ops.gated_delta_rule(xc, a_raw, x[:, C + ra + rg:], g_raw, P["A_log"].to(dev), P["dt_bias"].to(dev),
                                   P["norm"].to(dev), state, qsl, lens_now, tbl, H, G, D, E, eps).cpu()
        o = 0
        for s, n in order:
            got[s].append(out[o:o + n])
            o += n
            done[s] += n
    for s in range(2):
        assert done[s] == lens[s]
        torch.testing.assert_close(torch.cat(got[s]), want[s], atol=3e-5, rtol=3e-4)


# ---- whole models through the engine --------------------------------------------------------------------------------
VARIANTS = {
    "hybrid": dict(layers=hybrid_layers()),
    "plain_residual": dict(layers=hybrid_layers()[:2], streams=None),
    "three_streams_no_cap": dict(layers=hybrid_layers()[1:3], streams=3, softcap=None),
    "one_stream": dict(layers=hybrid_layers()[:2], streams=1, embed_scale=1.0),
    "no_feed_forward": dict(layers=[O.attention_layer(ff=None), O.delta_layer(ff=None), O.attention_layer()]),
    "attention_only_no_mask": dict(layers=[O.attention_layer(window=None), O.attention_layer(heads=1, kv_heads=1,
                                                                                           keep_first=0)]),
    "delta_only_taps": dict(layers=[O.delta_layer(conv=2), O.delta_layer(heads=4, kv_heads=1, dim=20, vdim=12, conv=5)]),
}


@pytest.mark.parametrize("dev,dtype", CASES)
@pytest.mark.parametrize("name", list(VARIANTS))
def test_whole_prompt(tmp_path, dev, dtype, name):
    kw = dict(VARIANTS[name])
    folder, cfg, W = model(tmp_path, kw.pop("layers"), seed=3, **kw)
    prompts = {"a": tokens(45, cfg["vocab"], 1), "b": tokens(1, cfg["vocab"], 2)}
    got = run_schedule(folder, dtype, dev, prompts, [[("a", 45)], [("b", 1)]], 64)
    check(cfg, W, prompts, got, dtype)


@pytest.mark.parametrize("dev,dtype", CASES)
def test_decode_token_by_token_past_the_window(tmp_path, dev, dtype):
    folder, cfg, W = model(tmp_path, hybrid_layers(), seed=4, sharp=True)
    p = tokens(70, cfg["vocab"], 5)
    sched = [[("a", 11)]] + [[("a", 1)]] * 59          # decodes 59 tokens: five windows of 12, nine of 7
    got = run_schedule(folder, dtype, dev, {"a": p}, sched, 80)
    check(cfg, W, {"a": p}, got, dtype)


@pytest.mark.parametrize("dev,dtype", CASES)
@pytest.mark.parametrize("block_size", [16, 32])
def test_portions_down_to_two_tokens(tmp_path, dev, dtype, block_size):
    folder, cfg, W = model(tmp_path, hybrid_layers(), seed=6, sharp=True)
    p = tokens(90, cfg["vocab"], 7)
    cuts = [2, 3, 11, 2, 16, 1, 17, 2, 7, 12, 1, 1, 15]
    assert sum(cuts) == 90
    got = run_schedule(folder, dtype, dev, {"a": p}, [[("a", n)] for n in cuts], 96, block_size=block_size)
    check(cfg, W, {"a": p}, got, dtype)


@pytest.mark.parametrize("dev,dtype", CASES)
def test_unequal_requests_share_steps_and_reuse_pages_and_slots(tmp_path, dev, dtype):
    """Seven requests over four slots and a pool of 10 pages: portions beside single tokens, requests that sit out
    steps, pages and slots of finished requests taken by later ones."""
    folder, cfg, W = model(tmp_path, hybrid_layers(), seed=8, sharp=True)
    V = cfg["vocab"]
    prompts = {"a": tokens(40, V, 1), "b": tokens(17, V, 2), "c": tokens(1, V, 3), "d": tokens(33, V, 4),
               "e": tokens(48, V, 5), "f": tokens(9, V, 6), "g": tokens(30, V, 7)}
    sched = [[("a", 13), ("b", 2)], [("a", 1), ("b", 15), ("c", 1)], [("a", 20), ("d", 16)],
             [("d", 1), ("a", 1)], [("a", 5), ("d", 16)],                       # a, b, c, d done: their pages return
             [("e", 31), ("f", 2)], [("e", 1), ("f", 1), ("g", 2)], [("g", 28), ("e", 1)],
             [("e", 15), ("f", 6)]]
    got = run_schedule(folder, dtype, dev, prompts, sched, 160)
    check(cfg, W, prompts, got, dtype)


@pytest.mark.parametrize("dev,dtype", CASES)
def test_far_key_and_edges_that_matter(tmp_path, dev, dtype):
    """One attention layer whose weights make a single 'needle' token dominate: its key matches every later query
    and everything else is switched off by the bias, so the output changes by O(1) exactly where the needle enters
    or leaves the window or the kept prefix; the delta layer must carry the needle over hundreds of tokens."""
    layers = [O.attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=40, keep_first=3, ff=None, scale=1.0),
              O.delta_layer(heads=2, kv_heads=2, dim=16, vdim=16, ff=None)]
    cfg = O.make_config(layers, vocab=64, width=32, streams=2)
    W = O.make_weights(cfg, 11)
    # token 0 is the needle: alone along e0.  Every other token is mostly e2, which turns into a query along the
    # needle's key direction (head dim 0) and into a key along head dim 1.
    emb = 0.2 * W["embed"].float()
    emb[:, 0] = 0
    emb[:, 2] = 3.0
    emb[0] = 0
    emb[0, 0] = 6.0
    W["embed"] = emb.to(torch.bfloat16)
    q = torch.zeros(32, 32)
    q[0, 2] = q[16, 2] = 1.0
    k = torch.zeros(16, 32)
    k[0, 0], k[1, 2] = 1.0, 0.5
    W["l0.mix.q"], W["l0.mix.k"] = q.to(torch.bfloat16), k.to(torch.bfloat16)
    W["l0.mix.pb"] = torch.tensor([-8.0, -8.0]).to(torch.bfloat16)
    W["l0.mix.talk"] = torch.eye(2).to(torch.bfloat16)
    W["l1.mix.A_log"] = torch.tensor([-6.0, -5.0]).to(torch.bfloat16)       # a state that forgets slowly
    folder = O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    V = cfg["vocab"]
    body = [t % (V - 1) + 1 for t in tokens(400, V, 12)]
    prompts = {"sink": [0] + body[:150],            # needle inside the kept prefix: seen for ever
               "edge": body[:3] + [0] + body[3:120],          # needle just behind the kept prefix: leaves after a window
               "far": body[:50] + [0] + body[50:330]}         # needle far back for the recurrent layer
    sched = [[("sink", 100), ("edge", 30)], [("sink", 1), ("edge", 1)], [("sink", 50), ("edge", 10)],
             [("edge", 1)], [("edge", 1)], [("edge", 1)], [("edge", 1)], [("edge", 76), ("far", 200)],
             [("far", 129)], [("far", 1)], [("far", 1)]]
    got = run_schedule(folder, dtype, dev, prompts, sched, 560)
    check(cfg, W, prompts, got, dtype)
    # the crafted edge is real: hiding the needle one token early changes the logits there
    full = O.forward(cfg, W, prompts["edge"])
    cfg2 = O.make_config([dict(layers[0], mixer=dict(layers[0]["mixer"], mask={"size": 39, "keep_first": 3})), layers[1]],
                         vocab=64, width=32, streams=2)
    assert O.logit_error(O.forward(cfg2, W, prompts["edge"])[42], full[42]) > 0.3
    cfg3 = O.make_config([dict(layers[0], mixer=dict(layers[0]["mixer"], mask={"size": 40, "keep_first": 4})), layers[1]],
                         vocab=64, width=32, streams=2)
    assert O.logit_error(O.forward(cfg3, W, prompts["edge"])[100], full[100]) > 0.3


@pytest.mark.parametrize("dev", DEVICES)
def test_greedy_generation_through_llm(tmp_path, dev):
    """The engine's own entry point and scheduler: greedy continuation of three prompts of unequal length equals
    the oracle's (recomputed from scratch for every token)."""
    from vllm_distributed_amd import LLM, SamplingParams
    folder, cfg, W = model(tmp_path, hybrid_layers(), seed=9)
    V = cfg["vocab"]
    prompts = [tokens(19, V, 1), tokens(3, V, 2), tokens(33, V, 3)]
    llm = LLM(model=folder, skip_tokenizer_init=True, dtype="float32", device=dev, max_model_len=128, max_num_seqs=4,
              max_num_batched_tokens=24, enable_chunked_prefill=True, gpu_memory_utilization=0.1, enforce_eager=True)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(temperature=0, max_tokens=10,
                                                                                 ignore_eos=True))
    llm.shutdown()
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.outputs[0].token_ids:
            logits = O.forward(cfg, W, seq)[-1]
            best = int(logits.argmax())
            assert tok == best or logits[best] - logits[tok] < 1e-3, (len(seq), tok, best)
            seq.append(tok)
        assert len(o.outputs[0].token_ids) == 10


@pytest.mark.gpu
def test_decode_graphs_equal_eager(tmp_path):
    """Single decoded tokens through captured graphs (several replays with other work between them) give the
    eager logits."""
    folder, cfg, W = model(tmp_path, hybrid_layers(), seed=10)
    V = cfg["vocab"]
    prompts = {"a": tokens(30, V, 1), "b": tokens(22, V, 2)}
    sched = [[("a", 10), ("b", 4)]] + [[("a", 1), ("b", 1)]] * 18 + [[("a", 2)]]
    eager = run_schedule(folder, "bfloat16", "cuda", prompts, sched, 64, eager=True)
    graph = run_schedule(folder, "bfloat16", "cuda", prompts, sched, 64, eager=False)
    for k in prompts:
        torch.testing.assert_close(graph[k], eager[k], atol=1e-3, rtol=1e-3)
    check(cfg, W, prompts, graph, "bfloat16")
