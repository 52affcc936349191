"""Sapapel through the framework (checkpoint loader, scheduler, block manager and state slots,
model runner, kernels) against the plain per-sequence model of tests/oracle_sapapel.py.

Every test builds its own small configuration and random weights, writes them as a checkpoint
folder and loads that through the engine.  The same tests run on the CPU (the ops' PyTorch
compositions) and, marked gpu, on the HIP kernels."""
import json
import math
import os
import random
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import oracle_sapapel as O  # noqa: E402

from polykey_service_amd.engine import EngineConfig, LLMEngine, SamplingParams  # noqa: E402
from polykey_service_amd.parallel.state import ParallelState  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 32


def checkpoint(tmp_path, cfg, w, name="m"):
    from safetensors.torch import save_file
    d = tmp_path / name
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    return str(d)


def engine(path, device, dtype="float32", pool_tokens=512, max_seqs=4, budget=512, graphs=False):
    cfg = EngineConfig(model_path=path, dtype=dtype, block_size=BS, max_num_seqs=max_seqs, max_num_batched_tokens=budget,
                       max_model_len=pool_tokens, num_kv_blocks=pool_tokens // BS, watermark=0.0, hip_graphs=graphs,
                       device=device, graph_batch_sizes=(1, 2, 4))
    return LLMEngine(cfg, ParallelState(device=torch.device(device)))


def replay(eng, steps):
    """steps: list of lists of (id, tokens, want, end?) -> {id: {position: logits row}}."""
    got, at = {}, {}
    for step in steps:
        ends = [e[0] for e in step if len(e) > 3 and e[3]]
        lg = eng.replay_step([(e[0], e[1], e[2]) for e in step], ends)
        r = 0
        for e in step:
            base = at.get(e[0], 0)
            for wpos in e[2]:
                got.setdefault(e[0], {})[base + wpos] = lg[r]
                r += 1
            at[e[0]] = base + len(e[1])
            if e[0] in ends:
                at.pop(e[0])
    return got


def cut(rid, toks, sizes, end=True):
    """The request in portions of the given sizes (the rest one token at a time), all places wanted."""
    out, i = [], 0
    sizes = list(sizes)
    while i < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - i)
        out.append((rid, toks[i:i + n], list(range(n)), end and i + n == len(toks)))
        i += n
    return out


def close(a, b, tol=2e-4):
    torch.testing.assert_close(a, b, rtol=tol, atol=tol)


def rand_tokens(n, vocab, seed):
    return random.Random(seed).choices(range(vocab), k=n)


@pytest.fixture
def small(tmp_path):
    cfg = O.make_config(vocab=96, width=48, layers=3, heads=3, dim=8, vdim=12, kv_rank=20, ff=40, experts=5, top=2,
                        alpha=2.0, eps=1e-5)
    w = O.random_model(cfg, seed=3)
    return cfg, w, checkpoint(tmp_path, cfg, w)


# ------------------------------------------------------------------ each mechanism alone
def test_norm_shift_depth_ops_match_the_equations():
    from polykey_service_amd.ops import stream
    torch.manual_seed(1)
    W, n = 40, 9
    x, y, g = torch.randn(n, W), torch.randn(n, W), torch.tensor([0.7])
    out, _ = stream.sum_gain_norm(x, y, 3.0, g, 1e-5, out=torch.zeros(n, W))
    close(out, O.gain_rms_norm(3.0 * x + y, g, 1e-5), 1e-5)
    # the average over earlier outputs: entry nh-1 is this layer's normed sum
    hist = torch.randn(4, n, W)
    coef = torch.randn(4)
    want = sum(coef[j] * hist[j] for j in range(2)) + coef[2] * O.gain_rms_norm(3.0 * x + y, g, 1e-5)
    out, _ = stream.sum_gain_norm(x, y, 3.0, g, 1e-5, out=torch.zeros(n, W), hist=hist, nh=3, coef=coef)
    close(out, want, 1e-5)
    # token shift over one sequence cut 4 + 1 + 4, the previous row carried in a state slot
    mu = torch.rand(W)
    want = O.token_shift(x, mu)
    state = torch.full((3, W), 7.0)  # a slot used before: position 0 must not read it
    got, pos = [], 0
    for a, b in ((0, 4), (4, 5), (5, 9)):
        T = b - a
        meta = dict(token_seq=torch.zeros(T, dtype=torch.int32), cu_q=torch.tensor([0, T], dtype=torch.int32),
                    positions=torch.arange(a, b, dtype=torch.int32), slots=torch.tensor([1], dtype=torch.int32))
        got.append(stream.token_shift(x[a:b].contiguous(), mu, state, meta["token_seq"], meta["cu_q"], meta["positions"],
                                      meta["slots"], torch.float32))
        stream.save_last_rows(x[a:b].contiguous(), state, meta["cu_q"], meta["slots"], 1)
    close(torch.cat(got), want, 1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,V,R", [(3, 8, 12, 20), (1, 16, 4, 33), (4, 4, 4, 8)])
def test_latent_attention_mixer(device, H, D, V, R):
    from polykey_service_amd.models.config import LatentAttentionSpec
    from polykey_service_amd.models.sapapel import LatentAttention
    from polykey_service_amd.ops.attention import AttnMetadata
    torch.manual_seed(2)
    W, n, dev = 40, 70, torch.device(device)
    spec = {"heads": H, "dim": D, "vdim": V, "kv_rank": R, "scale": 0.3}
    w = {k: torch.randn(*s) * 0.2 for k, s in {"q": (H * D, W), "dkv": (R, W), "uk": (H * D, R), "uv": (H * V, R),
                                               "g": (H * V, W), "o": (W, H * V)}.items()}
    w["dkv.norm"] = 1 + 0.1 * torch.randn(R)
    h = torch.randn(n, W)
    want = O.latent_attention(h, w, "", spec, 1e-5)
    mix = LatentAttention(LatentAttentionSpec(H, D, V, R, 0.3), W)
    mix.set(w["q"], w["dkv"], w["dkv.norm"], w["uk"], w["uv"], w["g"], w["o"], torch.float32, dev)
    cache = torch.zeros(8, BS, R, device=dev)
    table = torch.tensor([[5, 2, 7, 0]], dtype=torch.int32, device=dev)
    got = []
    for a, b in ((0, 31), (31, 33), (33, 34), (34, 70)):  # portions across the page borders at 32 and 64
        pos = torch.arange(a, b)
        md = AttnMetadata(0, 1, b - a, b - a, (table[0].cpu()[pos // BS] * BS + pos % BS).to(torch.int32).to(dev))
        md.num_seqs, md.block_tables, md.num_decode = 1, table, 0
        md.cu_q = torch.tensor([0, b - a], dtype=torch.int32, device=dev)
        md.context_lens = torch.tensor([b], dtype=torch.int32, device=dev)
        got.append(mix(h[a:b].to(dev), md, cache, 1e-5).cpu())
    close(torch.cat(got), want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["first", "page_last", "page_first", "self", "next"])
def test_attention_finds_one_far_key(device, where):
    """One key's score stands far above the rest: the output is that key's latent when the key is
    visible (first token, either side of a page border, the query's own), and is untouched by it
    when the key is the query's successor in the same portion."""
    from polykey_service_amd.ops import latent_attention as la
    torch.manual_seed(5)
    dev, R, ctx, qn = torch.device(device), 24, 300, 7
    pool = torch.randperm(12)
    table = pool[:10].to(torch.int32).view(1, -1)
    c = torch.randn(ctx, R) * 0.1
    qpos = ctx - 3  # a query in the middle of the last portion
    key = {"first": 0, "page_last": 3 * BS - 1, "page_first": 3 * BS, "self": qpos, "next": qpos + 1}[where]
    q = torch.randn(2, qn, R) * 0.1
    q[:, qpos - (ctx - qn)] = 40.0 * c[key] / c[key].norm()
    c[key] = c[key] / c[key].norm() * 4.0
    cache = torch.zeros(12, BS, R)
    idx = torch.arange(ctx)
    cache.view(-1, R)[table[0].long()[idx // BS] * BS + idx % BS] = c
    out = la.latent_attention(q.to(dev), cache.to(dev), table.to(dev), torch.tensor([0, qn], dtype=torch.int32, device=dev),
                              torch.tensor([ctx], dtype=torch.int32, device=dev), 1, 1.0).cpu()
    row = out[0, qpos - (ctx - qn)]
    if where == "next":
        sc = (c[:qpos + 1] @ q[0, qpos - (ctx - qn)])
        close(row, torch.softmax(sc, 0) @ c[:qpos + 1], 1e-4)
        assert (row - c[key]).norm() > 1.0
    else:
        close(row, c[key], 1e-3)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,F", [(5, 2, 40), (3, 1, 17), (4, 4, 8), (70, 3, 12)])
def test_sigmoid_moe_block(device, E, top, F):
    from polykey_service_amd.models.config import SigmoidMoESpec
    from polykey_service_amd.models.sapapel import SigmoidMoE
    torch.manual_seed(4)
    W, n, dev = 40, 45, torch.device(device)
    w = {"router": torch.randn(E, W) * 0.4}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = torch.randn(F, W) * 0.2, torch.randn(F, W) * 0.2, torch.randn(W, F) * 0.2
    x = torch.randn(n, W)
    want = O.sigmoid_moe(x, w, "", {"router": {"experts": E, "top": top}})
    blk = SigmoidMoE(SigmoidMoESpec(E, top, F))
    blk.set(w["router"], [w[f"e{e}.gate"] for e in range(E)], [w[f"e{e}.up"] for e in range(E)],
            [w[f"e{e}.down"] for e in range(E)], torch.float32, dev)
    close(blk(x.to(dev), x.to(dev)).cpu(), want, 1e-4)


def test_router_prefers_the_lower_expert_on_equal_scores():
    from polykey_service_amd.ops import moe
    rw = torch.randn(4, 16)
    rw[2] = rw[0]
    x = rw[0][None] * 3
    ids, s = moe.route_sigmoid_topk(x, rw, 2)
    assert ids.tolist() == [[0, 2]] and float(s[0, 0]) == float(s[0, 1])


# ------------------------------------------------------------------ whole model through the engine
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_matches_decoding_token_by_token(device, small):
    cfg, w, path = small
    toks = rand_tokens(75, cfg["vocab"], 1)
    want = O.forward(toks, w, cfg)
    eng = engine(path, device)
    whole = replay(eng, [[("a", toks, list(range(75)), True)]])["a"]
    single = replay(eng, [[s] for s in cut("b", toks, [])])["b"]
    for p in range(75):
        close(whole[p], want[p])
        close(single[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 30, 3, 31], [33, 2, 29, 2], [64, 2], [5, 1, 1, 60]])
def test_portions_of_any_size(device, small, sizes):
    cfg, w, path = small
    toks = rand_tokens(70, cfg["vocab"], 2)
    want = O.forward(toks, w, cfg)
    got = replay(engine(path, device), [[s] for s in cut("a", toks, sizes)])["a"]
    for p in range(70):
        close(got[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_match_each_request_alone(device, small):
    cfg, w, path = small
    V = cfg["vocab"]
    reqs = {"a": rand_tokens(90, V, 10), "b": rand_tokens(40, V, 11), "c": rand_tokens(3, V, 12), "d": rand_tokens(66, V, 13),
            "e": rand_tokens(1, V, 14), "f": rand_tokens(35, V, 15)}
    want = {k: O.forward(t, w, cfg) for k, t in reqs.items()}
    plans = {"a": cut("a", reqs["a"], [31, 2, 40]), "b": cut("b", reqs["b"], [2, 30]), "c": cut("c", reqs["c"], [3]),
             "d": cut("d", reqs["d"], [64]), "e": cut("e", reqs["e"], [1]), "f": cut("f", reqs["f"], [20, 2])}
    # a, b, c, d start together (four live requests); e and f take the slots and pages that c and b free
    steps, live, queue = [], ["a", "b", "c", "d"], ["e", "f"]
    n = 0
    while live:
        step = []
        for k in list(live):
            if k == "d" and n % 3 == 1 and plans[k]:
                continue  # sits out a step
            step.append(plans[k].pop(0))
            if not plans[k]:
                live.remove(k)
                if queue:
                    live.append(queue.pop(0))
        steps.append(step)
        n += 1
    eng = engine(path, device, pool_tokens=320)  # 10 pages: less than the requests' sum of 13
    got = replay(eng, steps)
    for k, t in reqs.items():
        for p in range(len(t)):
            close(got[k][p], want[k][p])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_are_reused(device, small):
    cfg, w, path = small
    eng = engine(path, device, pool_tokens=128, max_seqs=2)
    for i in range(5):  # every request lands on pages and a slot that another one just left
        toks = rand_tokens(50 + 7 * i, cfg["vocab"], 20 + i)
        want = O.forward(toks, w, cfg)
        got = replay(eng, [[s] for s in cut(f"r{i}", toks, [30 + i, 2])])[f"r{i}"]
        for p in (0, 1, 29 + i, 30 + i, 32, len(toks) - 1):
            close(got[p], want[p])
    with pytest.raises(RuntimeError):  # a third live request has no state slot
        eng.replay_step([("x", [1, 2], []), ("y", [1, 2], []), ("z", [1, 2], [])], [])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_across_pages(device, small):
    cfg, w, path = small
    toks = rand_tokens(140, cfg["vocab"], 30)
    want = O.forward(toks, w, cfg)
    got = replay(engine(path, device), [[s] for s in cut("a", toks, [20])])["a"]
    for p in list(range(18, 24)) + [31, 32, 63, 64, 65, 95, 96, 127, 128, 139]:
        close(got[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [
    dict(width=40, heads=1, dim=16, vdim=4, kv_rank=33, ff=17, experts=3, top=1, alpha=1.0, layers=2),
    dict(width=64, heads=4, dim=4, vdim=4, kv_rank=8, ff=8, experts=4, top=4, alpha=0.5, layers=1, eps=1e-3),
    dict(width=56, heads=2, dim=24, vdim=8, kv_rank=16, ff=30, experts=70, top=3, layers=4, mlp_none=(1, 3), scale=0.05),
])
def test_other_sizes(device, tmp_path, kw):
    cfg = O.make_config(vocab=50, **kw)
    w = O.random_model(cfg, seed=7)
    if kw.get("layers") == 4:  # a layer without shift, one without depth weights; of the two layers
        del w["l2.shift"], w["l0.dwa"]  # without feed-forward, one still has its second norm
        w["l3.norm2"] = torch.tensor(1.25)
    path = checkpoint(tmp_path, cfg, w)
    toks = rand_tokens(45, 50, 3)
    want = O.forward(toks, w, cfg)
    got = replay(engine(path, device), [[s] for s in cut("a", toks, [7, 2, 30])])["a"]
    for p in range(45):
        close(got[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_stays_near_the_fp32_model(device, small):
    cfg, w, path = small
    toks = rand_tokens(60, cfg["vocab"], 5)
    want = O.forward(toks, w, cfg)
    got = replay(engine(path, device, dtype="bfloat16"), [[s] for s in cut("a", toks, [40, 2])])["a"]
    err = torch.stack([got[p] - want[p] for p in range(60)])
    assert float(err.pow(2).mean().sqrt()) < 0.05 * float(want.pow(2).mean().sqrt())


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device, small):
    """LLMEngine.generate: the scheduler's own batching (chunked prefill under a small budget,
    mixed steps, decode graphs on the GPU) yields the plain model's greedy continuation."""
    cfg, w, path = small
    prompts = [rand_tokens(n, cfg["vocab"], 40 + n) for n in (50, 3, 21)]
    want = []
    for pr in prompts:
        seq = list(pr)
        for _ in range(12):
            lg = O.forward(seq, w, cfg)[-1]
            top2 = lg.topk(2).values
            assert float(top2[0] - top2[1]) > 1e-3  # no near-tie that rounding could flip
            seq.append(int(lg.argmax()))
        want.append(seq[len(pr):])
    eng = engine(path, device, budget=32, graphs=device == "cuda")
    got = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    assert got == want
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4
    if device == "cuda":
        assert eng.runner.stats["graph_steps"] > 0


@pytest.mark.gpu
def test_pipelined_decode_continuations(small):
    """Overlapped engine steps: decode step k+1 is launched from step k's sampled ids while they are
    still on the GPU (graph replays); the tokens equal the unpipelined engine's."""
    cfg, w, path = small
    prompts = [rand_tokens(n, cfg["vocab"], 60 + n) for n in (40, 7)]

    def run(overlap):
        ecfg = EngineConfig(model_path=path, dtype="float32", block_size=BS, max_num_seqs=4, max_num_batched_tokens=256,
                            max_model_len=512, num_kv_blocks=16, watermark=0.0, hip_graphs=True, device="cuda",
                            graph_batch_sizes=(1, 2, 4), overlap=overlap)
        eng = LLMEngine(ecfg, ParallelState(device=torch.device("cuda")))
        out = eng.generate(prompts, SamplingParams(max_tokens=24, ignore_eos=True))
        return out, eng.continuation_steps

    plain, _ = run(False)
    piped, n_cont = run(True)
    assert piped == plain and n_cont > 0


@pytest.mark.gpu
def test_aligned_sizes_on_the_matrix_core_paths(tmp_path):
    """Sizes that every fast path tiles (bf16): MFMA latent attention for prompts and decoding with
    the latent-major cache copy, grouped MFMA expert GEMMs on scaled rows, split-K decode
    projections summed inside the norm kernel.  Against the fp32 model within bf16 rounding, for a
    prompt in portions, decoded tokens, and a second request sharing the steps."""
    cfg = O.make_config(vocab=128, width=256, layers=2, heads=2, dim=64, vdim=128, kv_rank=128, ff=256, experts=4, top=2)
    w = O.random_model(cfg, seed=11, std=0.04)
    path = checkpoint(tmp_path, cfg, w)
    eng = engine(path, "cuda", dtype="bfloat16")
    eng.runner.cfg.hip_graphs = True  # decode graphs whose logits stay readable, as bin/trace_run captures them
    eng.runner.capture_graphs([1, 2, 4], keep_logits=True)
    L = eng.model.layers[0]
    assert L.mlp.w13 is not None and L.mlp.w13_p is not None and L.mix.w_o_p is not None
    assert eng.runner.kv_caches[0][1] is not None  # the latent-major copy
    a, b = rand_tokens(150, 128, 1), rand_tokens(40, 128, 2)
    want = {"a": O.forward(a, w, cfg), "b": O.forward(b, w, cfg)}
    pa, pb = cut("a", a, [70, 2, 50]), cut("b", b, [33])
    steps = [[pa.pop(0)]] + [[x, y] for x, y in zip(pa, pb)] + [[x] for x in pa[len(pb):]]
    got = replay(eng, steps)
    assert eng.runner.stats["graph_steps"] > 0
    for k, toks in (("a", a), ("b", b)):
        err = torch.stack([got[k][p] - want[k][p] for p in range(len(toks))])
        assert float(err.pow(2).mean().sqrt()) < 0.04 * float(want[k].pow(2).mean().sqrt())
        assert float(err.abs().max()) < 0.25 * float(want[k].abs().max())


def test_served_over_grpc_with_sampling(small):
    """The family behind the gRPC tool surface (AsyncLLM loop, tokenizer, sampler): greedy ids equal
    the plain model's continuation, seeded sampling is reproducible and uses the state slots of
    several concurrent requests."""
    import grpc

    from polykey_service_amd import proto
    from polykey_service_amd.adapters.local_llm import attach_local_llm
    from polykey_service_amd.config.server_config import ServerConfig
    from polykey_service_amd.service import ToolRouter
    from polykey_service_amd.utils import slog
    from tests.helpers import ServerThread

    cfg, w, path = small
    eng = LLMEngine(EngineConfig(model_path=path, dtype="float32", max_num_seqs=4, max_num_batched_tokens=64,
                                 max_model_len=256, num_kv_blocks=32, hip_graphs=False, device="cpu"), ParallelState())
    router = ToolRouter()
    attach_local_llm(router, ServerConfig(model="m", model_path=path, backend="local"), slog.Logger(open(os.devnull, "w")),
                     engine=eng)
    prompt = rand_tokens(20, cfg["vocab"], 77)
    seq = list(prompt)
    for _ in range(6):
        seq.append(int(O.forward(seq, w, cfg)[-1].argmax()))

    def req(**params):
        r = proto.ExecuteToolRequest(tool_name="llm.generate")
        r.parameters.update(params)
        return r

    try:
        with ServerThread(router) as s, grpc.insecure_channel(s.addr) as ch:
            call = ch.unary_unary(proto.EXECUTE_TOOL, request_serializer=proto.ExecuteToolRequest.SerializeToString,
                                  response_deserializer=proto.ExecuteToolResponse.FromString)
            r = call(req(prompt_token_ids=prompt, max_tokens=6, ignore_eos=True, return_token_ids=True, **{"return": "struct"}), timeout=120)
            d = proto.struct_to_dict(r.struct_output)
            assert [int(t) for t in d["token_ids"]] == seq[len(prompt):], d
            futs = [call.future(req(prompt_token_ids=rand_tokens(9 + i, cfg["vocab"], i), max_tokens=5, temperature=0.8,
                                    top_p=0.9, seed=5, ignore_eos=True, return_token_ids=True, **{"return": "struct"}), timeout=120)
                    for i in range(4)]
            first = [proto.struct_to_dict(f.result().struct_output)["token_ids"] for f in futs]
            again = proto.struct_to_dict(call(req(prompt_token_ids=rand_tokens(9, cfg["vocab"], 0), max_tokens=5,
                                                  temperature=0.8, top_p=0.9, seed=5, ignore_eos=True,
                                                  return_token_ids=True, **{"return": "struct"}),
                                              timeout=120).struct_output)["token_ids"]
            assert again == first[0] and all(len(t) == 5 for t in first)
    finally:
        router.llm.shutdown()
    assert eng.bm.num_free_state_slots == 4
