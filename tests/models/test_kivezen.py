"""Kivezen through the framework (checkpoint loader, scheduler, block manager and state slots,
model runner, kernels) against the plain per-sequence model of tests/oracle_kivezen.py.

Every test builds its own small configuration and random weights, writes them as a checkpoint
folder and loads that through the engine, or drives one op with hand-made inputs.  The same
tests run on the CPU (the ops' PyTorch compositions) and, marked gpu, on the HIP kernels."""
import json
import os
import random
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import oracle_kivezen as O  # noqa: E402

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


def engine(path, device, dtype="float32", pool_tokens=512, max_seqs=4, budget=512, graphs=False, max_len=None):
    cfg = EngineConfig(model_path=path, dtype=dtype, block_size=BS, max_num_seqs=max_seqs, max_num_batched_tokens=budget,
                       max_model_len=max_len or pool_tokens, num_kv_blocks=pool_tokens // BS, watermark=0.0,
                       hip_graphs=graphs, device=device, graph_batch_sizes=(1, 2, 4))
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


def close(a, b, tol=3e-4):
    torch.testing.assert_close(a.float(), b.float(), rtol=tol, atol=tol)


def rand_tokens(n, vocab, seed):
    return random.Random(seed).choices(range(vocab), k=n)


def model_logits(cfg, w, toks):
    return O.forward(cfg, w, toks).float()


@pytest.fixture
def small(tmp_path):
    # lightning, attention + mixture, attention + dense, the middle two run twice
    cfg = O.make_config(vocab=90, width=48, pattern="lAaL", heads=4, kv_heads=2, dim=8, vdim=12, rot_dims=6,
                        lightning=(3, 6, 10), loop=(1, 3, 2), streams=3)
    w = O.random_model(cfg, seed=3)
    return cfg, w, checkpoint(tmp_path, cfg, w)


# ------------------------------------------------------------------ each mechanism alone
def test_rotation_tables_match_the_frequency_rule():
    from polykey_service_amd.ops import sink_attention as sa
    for dims, base, sc in [(8, 1000.0, None), (40, 30000.0, (6.0, 1024, 24.0, 1.5)), (6, 10.0, (2.0, 16, 4.0, 0.5)),
                           (16, 100.0, (8.0, 40, 2.0, 2.0))]:
        f, mag = sa.pair_frequencies(dims, base, sc)
        want, wmag = O.rotary_frequencies(dims, base, dict(zip(("factor", "original", "fast", "slow"), sc)) if sc else None)
        torch.testing.assert_close(f, want, rtol=1e-12, atol=0)
        assert abs(mag - wmag) < 1e-12
        tab = sa.rotation_table(70, f, mag, "cpu")
        ang = torch.arange(70, dtype=torch.float64)[:, None] * want
        close(tab[..., 0], torch.cos(ang) * wmag, 1e-6)
        close(tab[..., 1], torch.sin(ang) * wmag, 1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S,moe,shared,T,W", [(1, False, False, 9, 40), (2, True, True, 9, 40), (3, True, False, 9, 42),
                                              (8, False, False, 9, 40), (2, True, True, 1100, 2056), (3, False, False, 5, 4100)])
def test_hyper_step(device, S, moe, shared, T, W):
    """Closing one sublayer and opening the next equals the stream equations, for one and several
    streams, with a plain output row or a mixture's weighted rows and gated shared row, at widths
    that are and are not multiples of four and at prompt-sized and decode-sized token counts."""
    from polykey_service_amd.ops import hyper
    torch.manual_seed(S)
    dev, top = torch.device(device), 3
    xs = torch.randn(T, S, W)
    mix, a_out, a_in, nw = torch.eye(S) + 0.3 * torch.randn(S, S), torch.randn(S), torch.randn(S), 1 + 0.1 * torch.randn(W)
    if moe:
        rows = torch.randn(T * top, W)
        inv = torch.randperm(T * top).to(torch.int32)
        inv[5] = -1
        wts = torch.rand(T, top)
        y = hyper.ExpertSum(rows.to(dev), inv.to(dev), wts.to(dev), top)
        idx = inv.long().view(T, top)
        yv = (torch.where((idx >= 0)[..., None], rows[idx.clamp(min=0)], torch.zeros(())) * wts[..., None]).sum(1)
        if shared:
            sh, gate = torch.randn(T, W), torch.randn(T, 7)[:, 3]
            y.shared, y.gate = sh.to(dev), gate.to(dev)
            yv = yv + sh * torch.sigmoid(gate)[:, None]
    else:
        yv = torch.randn(T, W)
        y = yv.to(dev)
    new = torch.einsum("st,nsw->ntw", mix, xs) + a_out[None, :, None] * yv[:, None, :]
    u = torch.einsum("t,ntw->nw", a_in, new)
    want = O.rms_norm(u.double(), nw.double(), 1e-5).float()
    xd = xs.to(dev).clone()
    act, z32 = hyper.hyper_step(xd, y, (mix.to(dev), a_out.to(dev)), (a_in.to(dev), nw.to(dev)), 1e-5, torch.float32,
                                want_f32=True)
    close(xd.cpu(), new, 1e-5)
    close(act.cpu(), want, 1e-5)
    close(z32.cpu(), want, 1e-5)
    pick = torch.tensor([T - 2, 0, 3], dtype=torch.int32)
    act2, _ = hyper.hyper_step(xd, None, None, (a_in.to(dev), nw.to(dev)), 1e-5, torch.float32, rows=pick.to(dev))
    close(act2.cpu(), want[pick.long()], 1e-5)


def _attention_case(H, G, D, V, rot_dims, n, scaling, softcap, seed, scale=None):
    """A one-layer attention problem whose mixer input rows are the raw q | k | v themselves."""
    m = O.make_config(pattern="a", heads=H, kv_heads=G, dim=D, vdim=V, rot_dims=rot_dims, scaling=scaling,
                      softcap=softcap, scale=scale)["layers"][0]["mixer"]
    torch.manual_seed(seed)
    width = (H + G) * D + G * V
    eye = torch.eye(width, dtype=torch.float64)
    w = {"q": eye[:H * D], "k": eye[H * D:(H + G) * D], "v": eye[(H + G) * D:], "o": torch.eye(H * V, dtype=torch.float64),
         "temp": (1 + 0.3 * torch.randn(H)).double()}
    return m, w, torch.randn(n, width)


def _run_attention(dev, m, w, h, portions, pages, eps=1e-5, dtype=torch.float32):
    """The framework's two attention ops over a hand-made paged cache, the sequence fed in portions."""
    from polykey_service_amd.ops import sink_attention as sa
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    rot = m.get("rot")
    qk_t = v_t = None
    if rot:
        f, mag = sa.pair_frequencies(rot["dims"], rot["base"], tuple(rot["scaling"].values()) if rot.get("scaling") else None)
        qk_t = sa.rotation_table(n + 3, f, mag, dev)
        v_t = sa.rotation_table(n + 3, sa.pair_frequencies(V, rot["base"])[0], 1.0, dev)
    nb = max(pages) + 1
    kc, vc = torch.zeros(nb + 2, G, BS, D, device=dev, dtype=dtype), torch.zeros(nb + 2, G, V, BS, device=dev, dtype=dtype)
    table = torch.tensor([pages], dtype=torch.int32, device=dev)
    hs = (w["temp"] * m["scale"]).float().to(dev)
    outs, at = [], 0
    for c in portions:
        pos = torch.arange(at, at + c, dtype=torch.int32, device=dev)
        slots = torch.tensor([pages[p // BS] * BS + p % BS for p in range(at, at + c)], dtype=torch.int32, device=dev)
        q = sa.rope_norm_cache(h[at:at + c].to(dev).to(dtype), pos, slots, qk_t, v_t, kc, vc, H, G, D, V, eps)
        cu = torch.tensor([0, c], dtype=torch.int32, device=dev)
        ctx = torch.tensor([at + c], dtype=torch.int32, device=dev)
        outs.append(sa.sink_attention(q, kc, vc, table, cu, ctx, 1, pos, hs, float(m.get("softcap") or 0.0), 1.0, v_t,
                                      num_decode=1 if (c == 1 and at > 0) else 0).float().cpu())
        at += c
    return torch.cat(outs)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,V,rd", [(4, 2, 8, 12, 6), (3, 3, 16, 4, 16), (6, 1, 6, 34, 2), (2, 1, 24, 24, 0)])
def test_attention_mixer(device, H, G, D, V, rd):
    """Rotation (partial, scaled), unit norm, rotated values, temperature, cap and sink against the
    plain attention, prompt portions and single decoded tokens over shuffled pages."""
    m, w, h = _attention_case(H, G, D, V, rd, 75, (3.0, 64, 8.0, 1.0) if rd else None, 20.0 if D != 16 else 0.0, seed=H)
    if rd == 0:
        del m["rot"]
    want = O.attention(h.double(), w, "", m, 1e-5).float()
    got = _run_attention(torch.device(device), m, w, h, [31, 2, 33, 1, 1, 7], [5, 0, 3])
    close(got, want, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["first", "page_last", "page_first", "self", "next"])
@pytest.mark.parametrize("decoded", [False, True])
def test_attention_finds_one_far_key(device, where, decoded):
    """One key's score stands far above the rest, so the output is that key's value when it is
    visible (the first token, either side of a page border, the query's own) and shows no trace of
    it when the key is the query's successor; checked for a prompt portion and a decoded token."""
    H, G, D, V, n = 2, 1, 8, 6, 200
    m, w, h = _attention_case(H, G, D, V, 0, n, None, 30.0, seed=11, scale=6.0)
    del m["rot"]
    w["temp"] = torch.ones(H, dtype=torch.float64)
    qpos = n - 3
    key = {"first": 0, "page_last": 3 * BS - 1, "page_first": 3 * BS, "self": qpos, "next": qpos + 1}[where]
    u = torch.randn(D)
    h[qpos, :H * D] = u.repeat(H)                     # both heads ask for u
    h[key, H * D:(H + G) * D] = u                     # one key answers
    h[key, (H + G) * D:] = 50.0 * torch.ones(V)       # with a value nothing else has
    want = O.attention(h.double(), w, "", m, 1e-5).float()
    portions = [n - 8] + ([1] * 8 if decoded else [8])
    got = _run_attention(torch.device(device), m, w, h, portions, [6, 2, 4, 0, 5, 1, 3])
    close(got[qpos], want[qpos], 5e-4)
    if where == "next":
        assert float(got[qpos].abs().max()) < 10.0
    else:
        assert float(got[qpos].min()) > 25.0          # the capped score 27.6 against a few of the others: the key dominates


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V", [(8, 2, 64, 64), (4, 4, 128, 128), (6, 1, 64, 128), (20, 1, 128, 64)])
def test_matrix_core_attention(H, G, D, V):
    """bf16 at head sizes the MFMA kernels tile: prompt portions that end inside a 32-key tile, and
    decoded tokens whose keys are cut into runs, against the plain rule and the FMA kernels."""
    from polykey_service_amd.ops import native
    m, w, h = _attention_case(H, G, D, V, D // 2, 330, (3.0, 64, 8.0, 1.0), 20.0, seed=V, scale=0.6)
    h = h.bfloat16().float()
    want = O.attention(h.double(), w, "", m, 1e-5).float()
    pages = [9, 3, 0, 7, 5, 1, 8, 2, 6, 4, 10]
    portions = [150, 2, 37, 120] + [1] * 21
    got = _run_attention(torch.device("cuda"), m, w, h, portions, pages, dtype=torch.bfloat16)
    native.call("pkm_set_sink_mfma", 0)
    try:
        fma = _run_attention(torch.device("cuda"), m, w, h, portions, pages, dtype=torch.bfloat16)
    finally:
        native.call("pkm_set_sink_mfma", 1)
    scale = float(want.pow(2).mean().sqrt())
    assert float((got - want).pow(2).mean(-1).sqrt().max()) < 0.03 * scale
    assert float((got - fma).pow(2).mean(-1).sqrt().max()) < 0.03 * scale


@pytest.mark.parametrize("device", DEVICES)
def test_softmax_sink_takes_its_share(device):
    """With scores near zero the sink holds 1 / (keys + 1) of the weight: one key gives half its value."""
    m, w, h = _attention_case(1, 1, 4, 4, 0, 3, None, 0.0, seed=2, scale=1e-6)
    del m["rot"]
    w["temp"] = torch.ones(1, dtype=torch.float64)
    got = _run_attention(torch.device(device), m, w, h, [3], [1])
    v = h[:, 8:]
    close(got[0], v[0] / 2, 1e-4)
    close(got[2], v.sum(0) / 4, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,V", [(3, 6, 10), (1, 20, 3), (2, 33, 17)])
def test_lightning_mixer(device, H, D, V):
    """The recurrence in portions (state carried in a slot, a slot reused by a new sequence) against
    the token-by-token rule, and the gated norm behind it."""
    from polykey_service_amd.ops import lightning as li
    torch.manual_seed(D)
    dev, n, W = torch.device(device), 70, H * (2 * D + 2 * V)
    m = {"heads": H, "dim": D, "vdim": V, "decay": [0.9 - 0.3 * i / H for i in range(H)]}
    eye = torch.eye(W, dtype=torch.float64)
    w = {"q": eye[:H * D], "k": eye[H * D:2 * H * D], "v": eye[2 * H * D:2 * H * D + H * V], "g": eye[2 * H * D + H * V:],
         "o": torch.eye(H * V, dtype=torch.float64), "norm": (1 + 0.1 * torch.randn(H * V)).double()}
    state = torch.full((3, H, D, V), 7.0, device=dev)  # what an earlier owner left
    decay = torch.tensor(m["decay"], device=dev)
    for seq in range(2):
        h = torch.randn(n, W) * 0.7
        want = O.lightning(h.double(), w, "", m, 1e-5).float()
        at, outs = 0, []
        for c in [33, 2, 1, 1, 30, 3]:
            pos = torch.arange(at, at + c, dtype=torch.int32, device=dev)
            o = li.lightning_attention(h[at:at + c, :H * (2 * D + V)].to(dev), state, decay,
                                       torch.tensor([0, c], dtype=torch.int32, device=dev), 1, pos,
                                       torch.tensor([1], dtype=torch.int32, device=dev), H, D, V)
            outs.append(li.gated_rms_norm(o, w["norm"].float().to(dev), h[at:at + c, H * (2 * D + V):].to(dev), 1e-5,
                                          torch.float32).cpu())
            at += c
        close(torch.cat(outs), want, 2e-4)
    assert float((state[0] - 7.0).abs().max()) == 0.0 and float((state[2] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("device", DEVICES)
def test_lightning_remembers_a_far_token(device):
    """A head with decay 1 - 1e-3 still carries a token from 300 positions back; one with decay 0.5
    has lost it: the far token's value shows in the first head only."""
    from polykey_service_amd.ops import lightning as li
    dev, H, D, V, n = torch.device(device), 2, 4, 4, 330
    x = torch.full((n, H * (2 * D + V)), -20.0)       # silu(-20) ~ 0: silent tokens
    x[20, H * D:2 * H * D] = 5.0                      # token 20 writes k = 5 ...
    x[20, 2 * H * D:] = 3.0                           # ... with v = 3
    x[320, :H * D] = 2.0                              # token 320 asks
    state = torch.zeros(1, H, D, V, device=dev)
    decay = torch.tensor([0.999, 0.5], device=dev)
    outs, at = [], 0
    for c in [100, 150, 60, 2] + [1] * 18:
        pos = torch.arange(at, at + c, dtype=torch.int32, device=dev)
        outs.append(li.lightning_attention(x[at:at + c].to(dev), state, decay, torch.tensor([0, c], dtype=torch.int32, device=dev),
                                           1, pos, torch.zeros(1, dtype=torch.int32, device=dev), H, D, V).cpu())
        at += c
    o = torch.cat(outs).view(n, H, V)
    silu = lambda z: z / (1 + torch.exp(torch.tensor(-z)))
    want = float(0.999 ** 300 * D * silu(5.0) * silu(3.0) * silu(2.0))
    close(o[320, 0], torch.full((V,), want), 1e-3)
    assert float(o[320, 1].abs().max()) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,F,shared", [(5, 2, 10, 14), (3, 1, 17, 0), (4, 4, 8, 6), (70, 3, 12, 5)])
def test_clamped_moe_block(device, E, top, F, shared):
    from polykey_service_amd.models.config import ClampedMoESpec
    from polykey_service_amd.models.kivezen import ClampedMoE
    from polykey_service_amd.ops import hyper
    torch.manual_seed(E)
    dev, T, W = torch.device(device), 37, 24
    f = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": F, "limit": 0.8}}
    if shared:
        f["shared"] = {"ff": shared, "limit": 1.1}
    cfg = {"width": W, "vocab": 8, "layers": [{"type": "lightning", "mixer": {"heads": 1, "dim": 2, "vdim": 2, "decay": [0.5]}, "mlp": f}],
           "norm": {"eps": 1e-5}}
    w = {k[len("l0.mlp."):]: v for k, v in O.random_model(cfg, seed=E).items() if k.startswith("l0.mlp.")}
    x = torch.randn(T, W)
    want = O.moe_ff(x.double(), {k: v.double() for k, v in w.items()}, "", f).float()
    mod = ClampedMoE(ClampedMoESpec(E, top, F, 0.8, shared, 1.1))
    sh = (w["shared.sg"], w["shared.gate"], w["shared.up"], w["shared.down"]) if shared else None
    mod.set(w["router"], [w[f"e{e}.gate"] for e in range(E)], [w[f"e{e}.up"] for e in range(E)],
            [w[f"e{e}.down"] for e in range(E)], sh, torch.float32, dev)
    es = mod(x.to(dev), x.to(dev))
    xs = torch.zeros(T, 1, W, device=dev)
    one = torch.ones(1, device=dev)
    hyper.hyper_step(xs, es, (one.view(1, 1), one), None, 1e-5, torch.float32)
    close(xs[:, 0].cpu(), want, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_router_logits_are_fp32_dot_products(device):
    from polykey_service_amd.ops import moe
    dev = torch.device(device)
    for T, N, W in [(5, 17, 2048), (3, 4, 42), (300, 9, 64)]:
        x, w = torch.randn(T, W), torch.randn(N, W)
        close(moe.router_logits(x.to(dev), w.to(dev)).cpu(), (x.double() @ w.double().T).float(), 2e-5)


def test_router_prefers_the_lower_expert_on_equal_logits():
    from polykey_service_amd.ops import moe
    z = torch.tensor([[0.5, 2.0, 2.0, -1.0, 2.0]])
    ids, wts = moe.route_topk_softmax(z, 5, 2)
    assert ids.tolist() == [[1, 2]] and abs(float(wts[0, 0]) - 0.5) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
def test_dense_feed_forward_and_caps(device):
    from polykey_service_amd.models.kivezen import tanh_cap
    from polykey_service_amd.ops import moe
    dev = torch.device(device)
    z = torch.linspace(-6, 6, 101)
    close(moe.gelu_tanh(z.clone().to(dev)).cpu(), O.gelu_tanh(z.double()).float(), 1e-6)
    close(tanh_cap(z.clone().to(dev) * 10, 30.0).cpu(), 30 * torch.tanh(z * 10 / 30), 1e-5)
    gu = torch.randn(5, 64) * 3
    for il in (False, True):
        g, u = (gu.view(5, 2, 2, 16)[:, :, 0].reshape(5, 32), gu.view(5, 2, 2, 16)[:, :, 1].reshape(5, 32)) if il else (gu[:, :32], gu[:, 32:])
        want = g.clamp(max=1.5) * torch.sigmoid(1.702 * g.clamp(max=1.5)) * (u.clamp(-1.5, 1.5) + 1)
        close(moe.clamped_glu(gu.to(dev), 1.5, interleaved=il).cpu(), want, 1e-5)


# ------------------------------------------------------------------ whole model through the engine
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_matches_decoding_token_by_token(device, small):
    cfg, w, path = small
    toks = rand_tokens(75, cfg["vocab"], 1)
    want = model_logits(cfg, w, toks)
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
    want = model_logits(cfg, w, toks)
    got = replay(engine(path, device), [[s] for s in cut("a", toks, sizes)])["a"]
    for p in range(70):
        close(got[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_match_each_request_alone(device, small):
    cfg, w, path = small
    V = cfg["vocab"]
    reqs = {"a": rand_tokens(90, V, 10), "b": rand_tokens(40, V, 11), "c": rand_tokens(3, V, 12), "d": rand_tokens(66, V, 13),
            "e": rand_tokens(1, V, 14), "f": rand_tokens(35, V, 15)}
    want = {k: model_logits(cfg, w, t) for k, t in reqs.items()}
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
    eng = engine(path, device, pool_tokens=320, max_len=128)  # 10 pages: less than the requests' sum of 13
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
        want = model_logits(cfg, w, toks)
        got = replay(eng, [[s] for s in cut(f"r{i}", toks, [30 + i, 2])])[f"r{i}"]
        for p in (0, 1, 29 + i, 30 + i, 32, len(toks) - 1):
            close(got[p], want[p])
    with pytest.raises(RuntimeError):  # a third live request has no state slot
        eng.replay_step([("x", [1, 2], []), ("y", [1, 2], []), ("z", [1, 2], [])], [])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_across_pages(device, small):
    cfg, w, path = small
    toks = rand_tokens(140, cfg["vocab"], 30)
    want = model_logits(cfg, w, toks)
    got = replay(engine(path, device), [[s] for s in cut("a", toks, [20])])["a"]
    for p in list(range(18, 24)) + [31, 32, 63, 64, 65, 95, 96, 127, 128, 139]:
        close(got[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [
    # one stream with its own coefficients, one head, no loop, a layer without feed-forward
    dict(width=40, pattern="Al", heads=1, kv_heads=1, dim=16, vdim=4, rot_dims=16, streams=1, experts=3, top=1,
         shared_ff=0, no_mlp=(1,), lightning=(1, 5, 7)),
    # the plain residual (no streams), top == experts, no caps, no scaling, every layer looped three times
    dict(width=64, pattern="aLA", heads=4, kv_heads=4, dim=4, vdim=4, streams=0, experts=4, top=4, expert_ff=8,
         softcap=0.0, logit_softcap=0.0, scaling=None, loop=(0, 3, 3), eps=1e-3),
    # many experts, many streams, wide values, a loop of one pass at the end
    dict(width=56, pattern="LaAl", heads=6, kv_heads=2, dim=10, vdim=34, rot_dims=4, streams=5, experts=70, top=3,
         loop=(2, 4, 1), lightning=(2, 24, 8), scale=0.7),
])
def test_other_sizes(device, tmp_path, kw):
    cfg = O.make_config(vocab=50, **kw)
    w = O.random_model(cfg, seed=7)
    if kw["width"] == 64:
        del w["l0.mix.temp"]  # a head temperature the checkpoint leaves out is 1
    path = checkpoint(tmp_path, cfg, w)
    toks = rand_tokens(45, 50, 3)
    want = model_logits(cfg, w, toks)
    got = replay(engine(path, device), [[s] for s in cut("a", toks, [7, 2, 30])])["a"]
    for p in range(45):
        close(got[p], want[p])


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_stays_near_the_fp32_model(device, small):
    cfg, w, path = small
    toks = rand_tokens(60, cfg["vocab"], 5)
    want = model_logits(cfg, w, toks)
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
            lg = model_logits(cfg, w, seq)[-1]
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
def test_aligned_sizes_on_the_matrix_core_paths(tmp_path):
    """bf16 at sizes the framework's MFMA GEMMs tile (width and expert size multiples of 256: grouped
    expert GEMMs, the weight-streaming decode GEMM): prompt portions, decoded tokens and a mixed
    batch stay within bf16 rounding of the plain model."""
    # every expert is chosen (top == experts), so bf16 rounding cannot move a token to another expert
    # width 512: decode projections run as split-K slabs, summed inside the kernels that read them
    cfg = O.make_config(vocab=512, width=512, pattern="LA", heads=4, kv_heads=2, dim=64, vdim=64, ff=512, experts=4, top=4,
                        expert_ff=256, shared_ff=256, limit=7.0, shared_limit=7.0, lightning=(4, 64, 64), streams=2)
    w = O.random_model(cfg, seed=9, std=0.05)
    path = checkpoint(tmp_path, cfg, w)
    a, b = rand_tokens(150, 512, 1), rand_tokens(70, 512, 2)
    want = {"a": model_logits(cfg, w, a), "b": model_logits(cfg, w, b)}
    eng = engine(path, "cuda", dtype="bfloat16", graphs=True)
    steps = [[("a", a[:100], list(range(100)))], [("a", a[100:140], list(range(40))), ("b", b[:64], list(range(64)))]]
    steps += [[("a", [a[140 + i]], [0], i == 9)] + ([("b", [b[64 + i]], [0], i == 5)] if i < 6 else []) for i in range(10)]
    got = replay(eng, steps)
    scale = float(want["a"].pow(2).mean().sqrt())
    for k, t in (("a", a), ("b", b)):
        err = torch.stack([got[k][p] - want[k][p] for p in range(len(t))]).pow(2).mean(-1).sqrt()
        # single tokens are several times more sensitive to bf16 rounding than the median one
        assert float(err.median()) < 0.015 * scale and float(err.max()) < 0.2 * scale, (k, err)
