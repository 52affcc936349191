"""HIP kernels of csrc/mixers against plain fp32 PyTorch (both element types, sizes that are not
multiples of any tile)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

from polykey_service_amd.ops import latent_attention as la
from polykey_service_amd.ops import moe, stream

DTYPES = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=2e-5, atol=2e-5) if dt == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def batch_meta(qlens, ctxs, bs, dev, nblocks=None, shuffle=True):
    """cu_q, context_lens, block tables over a shuffled pool, slots, positions, token_seq."""
    n = len(qlens)
    need = [math.ceil(c / bs) for c in ctxs]
    nblocks = nblocks or sum(need) + 3
    perm = torch.randperm(nblocks).tolist() if shuffle else list(range(nblocks))
    mb = max(need)
    bt = torch.zeros((n, mb), dtype=torch.int32)
    at = 0
    for s in range(n):
        for j in range(need[s]):
            bt[s, j] = perm[at]
            at += 1
    cu = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    pos, slots, tseq = [], [], []
    for s in range(n):
        for p in range(ctxs[s] - qlens[s], ctxs[s]):
            pos.append(p)
            slots.append(int(bt[s, p // bs]) * bs + p % bs)
            tseq.append(s)
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    return dict(cu_q=cu.to(dev), ctx=mk(ctxs), bt=bt.to(dev), pos=mk(pos), slots=mk(slots), tseq=mk(tseq), nblocks=nblocks)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [48, 200, 1024])
def test_embed_shift_save(dt, W):
    dev = torch.device("cuda")
    table = torch.randn(37, W).to(dt)
    ids = torch.randint(0, 37, (9,), dtype=torch.int32)
    out = torch.zeros(12, W)
    want = stream.embed_rows(table, ids, out.clone())
    got = stream.embed_rows(table.to(dev), ids.to(dev), out.to(dev))
    torch.testing.assert_close(got.cpu(), want)
    # three sequences: a first portion at position 0, a continued portion, a single decoded token
    m = batch_meta([4, 3, 1], [4, 10, 6], 4, torch.device("cpu"))
    x, mu, state = torch.randn(8, W), torch.rand(W), torch.randn(5, W)
    sl = torch.tensor([3, 0, 4], dtype=torch.int32)
    want = stream.token_shift(x, mu, state, m["tseq"], m["cu_q"], m["pos"], sl, dt)
    got = stream.token_shift(x.to(dev), mu.to(dev), state.to(dev), m["tseq"].to(dev), m["cu_q"].to(dev), m["pos"].to(dev),
                             sl.to(dev), dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    # position 0 never reads its slot
    torch.testing.assert_close(want[0].float(), (x[0] * (1 - mu)).to(dt).float(), **tol(dt))
    s_cpu, s_gpu = state.clone(), state.to(dev)
    stream.save_last_rows(x, s_cpu, m["cu_q"], sl, 3)
    stream.save_last_rows(x.to(dev), s_gpu, m["cu_q"].to(dev), sl.to(dev), 3)
    torch.testing.assert_close(s_gpu.cpu(), s_cpu)
    assert torch.equal(s_cpu[3], x[3]) and torch.equal(s_cpu[0], x[6]) and torch.equal(s_cpu[4], x[7])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [40, 333])
def test_sum_gain_norm(dt, W):
    dev = torch.device("cuda")
    T, L = 7, 3
    x, y = torch.randn(T, W), torch.randn(T, W).to(dt)
    g, coef = torch.tensor([1.3]), torch.randn(L + 1)
    hist = torch.randn(L + 1, 9, W)
    for kw in (dict(), dict(nh=3), dict(rows=torch.tensor([5, 0, 5], dtype=torch.int32)), dict(y=None)):
        nh = kw.get("nh", 0)
        rows = kw.get("rows")
        yy = kw.get("y", y)
        h_c, h_g = hist.clone(), hist.to(dev)
        R = T if rows is None else rows.numel()
        w_out, w_act = stream.sum_gain_norm(x, yy, 2.5, g, 1e-5, out=torch.zeros(R, W), act_dtype=dt, rows=rows,
                                            hist=h_c if nh else None, nh=nh, coef=coef if nh else None)
        g_out, g_act = stream.sum_gain_norm(x.to(dev), None if yy is None else yy.to(dev), 2.5, g.to(dev), 1e-5,
                                            out=torch.zeros(R, W, device=dev), act_dtype=dt,
                                            rows=None if rows is None else rows.to(dev), hist=h_g if nh else None, nh=nh,
                                            coef=coef.to(dev) if nh else None)
        torch.testing.assert_close(g_out.cpu(), w_out, rtol=2e-5, atol=2e-5)
        torch.testing.assert_close(g_act.cpu().float(), w_act.float(), **tol(dt))
        torch.testing.assert_close(h_g.cpu(), h_c, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,R,bs", [(3, 24, 4), (8, 96, 32), (5, 130, 32), (2, 520, 32)])
def test_latent_attention(dt, H, R, bs):
    dev = torch.device("cuda")
    qlens, ctxs = [5, 1, 37, 2], [5, 70, 37, 131]
    m = batch_meta(qlens, ctxs, bs, torch.device("cpu"))
    T = sum(qlens)
    cache = torch.randn(m["nblocks"], bs, R).to(dt)
    # the step's own latents are written first, through the norm + cache kernel
    dkv_wide = torch.randn(T, R + 9).to(dt)
    w = 1 + 0.1 * torch.randn(R)
    c_cpu, c_gpu = cache.clone(), cache.to(dev)
    la.latent_norm_cache(dkv_wide[:, 4:4 + R], w, 1e-5, c_cpu, m["slots"])
    la.latent_norm_cache(dkv_wide.to(dev)[:, 4:4 + R], w.to(dev), 1e-5, c_gpu, m["slots"].to(dev))
    torch.testing.assert_close(c_gpu.cpu().float(), c_cpu.float(), **tol(dt))
    q = (torch.randn(H, T, R) * 0.3).to(dt)
    want = la.latent_attention(q, c_cpu, m["bt"], m["cu_q"], m["ctx"], 4, 0.2)
    got = la.latent_attention(q.to(dev), c_cpu.to(dev), m["bt"].to(dev), m["cu_q"].to(dev), m["ctx"].to(dev), 4, 0.2)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    o, g = torch.randn(H, T, 12).to(dt), torch.randn(T, H * 12 + 5).to(dt)
    torch.testing.assert_close(la.gate_merge(o.to(dev), g.to(dev)[:, 5:]).cpu().float(),
                               la.gate_merge(o, g[:, 5:]).float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("E,k,F,W,T", [(5, 2, 40, 48, 19), (12, 1, 96, 200, 70), (70, 3, 33, 64, 50)])
def test_sigmoid_moe(dt, E, k, F, W, T):
    dev = torch.device("cuda")
    x = torch.randn(T, W)
    rw = torch.randn(E, W) * 0.3
    ids_c, w_c = moe.route_sigmoid_topk(x, rw, k)
    ids_g, w_g = moe.route_sigmoid_topk(x.to(dev), rw.to(dev), k)
    assert torch.equal(ids_g.cpu(), ids_c)
    torch.testing.assert_close(w_g.cpu(), w_c, rtol=1e-5, atol=1e-6)
    gate, up, down = (torch.randn(E, F, W) * 0.2).to(dt), (torch.randn(E, F, W) * 0.2).to(dt), (torch.randn(E, W, F) * 0.2).to(dt)
    xa = x.to(dt)
    want = moe.input_scaled_moe(x, xa, ids_c, w_c, gate, up, down)
    got = moe.input_scaled_moe(x.to(dev), xa.to(dev), ids_g, w_g, gate.to(dev), up.to(dev), down.to(dev))
    torch.testing.assert_close(got.cpu(), want, **(dict(rtol=1e-4, atol=1e-4) if dt == torch.float32 else tol(dt)))


def latent_major(cache):
    """[blocks, bs, R] -> [blocks, bs / 32, R, 32] with key k of a 32-key tile in column
    8 * ((k % 16) // 4) + k % 4 + 4 * (k // 16)."""
    nb, bs, R = cache.shape
    k = torch.arange(32)
    col = 8 * ((k % 16) // 4) + k % 4 + 4 * (k // 16)
    out = torch.zeros(nb, bs // 32, R, 32, dtype=cache.dtype)
    out[:, :, :, col] = cache.view(nb, bs // 32, 32, R).transpose(2, 3)
    return out


@pytest.mark.parametrize("H,R", [(8, 96), (16, 128), (5, 512), (3, 32), (20, 64)])
def test_latent_attention_matrix_core_kernels(H, R):
    """bf16 latents the MFMA kernels are built for: against the fp32 composition and against the
    FMA kernel on the same inputs; decoded tokens (decode kernel, runs merged) beside prompt
    portions over several row tiles, with and without the latent-major cache copy."""
    from polykey_service_amd.ops import native
    dev, bs = torch.device("cuda"), 32
    qlens, ctxs = [1, 1, 1, 70, 9, 33], [300, 31, 64, 70, 140, 97]
    m = batch_meta(qlens, ctxs, bs, torch.device("cpu"))
    T = sum(qlens)
    cache = (torch.randn(m["nblocks"], bs, R) * 0.7).bfloat16()
    q = (torch.randn(H, T, R) * 0.4).bfloat16()
    want = la.latent_attention(q, cache, m["bt"], m["cu_q"], m["ctx"], 6, R ** -0.5).float()
    args = (q.to(dev), cache.to(dev), m["bt"].to(dev), m["cu_q"].to(dev), m["ctx"].to(dev), 6, R ** -0.5)
    got = la.latent_attention(*args)
    got_t = la.latent_attention(*args, latent_major(cache).to(dev), 3)
    native.call("pkm_set_latent_mfma", 0)
    try:
        fma = la.latent_attention(*args)
    finally:
        native.call("pkm_set_latent_mfma", 1)
    for x in (fma, got, got_t):
        torch.testing.assert_close(x.cpu().float(), want, rtol=2e-2, atol=1e-2)
    assert not torch.equal(got, fma) or R == 32  # two kernels ran
    assert la.mfma_latent(R, torch.bfloat16, dev, bs) and not la.mfma_latent(R + 8, torch.bfloat16, dev, bs)


def test_norm_cache_writes_both_layouts():
    dev, bs, R = torch.device("cuda"), 64, 96
    m = batch_meta([70, 1], [70, 130], bs, torch.device("cpu"))
    dkv = torch.randn(71, R).bfloat16()
    w = 1 + 0.1 * torch.randn(R)
    c = torch.zeros(m["nblocks"], bs, R, dtype=torch.bfloat16, device=dev)
    c_t = la.alloc_latent_major(m["nblocks"], bs, R, dev)
    la.latent_norm_cache(dkv.to(dev), w.to(dev), 1e-5, c, m["slots"].to(dev), c_t)
    assert torch.equal(c_t.cpu(), latent_major(c.cpu())) and float(c.float().abs().sum()) > 0


@pytest.mark.parametrize("key", [0, 31, 32, 63, 64, 65, 500, 991])
def test_decode_kernel_finds_one_far_key(key):
    """A decoded token whose query matches ONE cached key (first key, either side of a page border,
    either side of a run border of the split context, the newest key): the output is that latent."""
    dev, bs, R, ctx = torch.device("cuda"), 32, 64, 992
    assert la.decode_runs(1024)[0] == 64  # keys 63 | 64 sit on a run border
    m = batch_meta([1], [ctx], bs, torch.device("cpu"))
    c = torch.randn(ctx, R) * 0.1
    c[key] = c[key] / c[key].norm() * 4.0
    q = (30.0 * c[key] / c[key].norm()).view(1, 1, R).repeat(3, 1, 1).bfloat16()
    cache = torch.zeros(m["nblocks"], bs, R)
    idx = torch.arange(ctx)
    cache.view(-1, R)[m["bt"][0].long()[idx // bs] * bs + idx % bs] = c
    cache = cache.bfloat16()
    out = la.latent_attention(q.to(dev), cache.to(dev), m["bt"].to(dev), m["cu_q"].to(dev), m["ctx"].to(dev), 1, 1.0,
                              latent_major(cache).to(dev), 1)
    torch.testing.assert_close(out[1, 0].cpu().float(), c[key].bfloat16().float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("E,k,F,W,T", [(4, 2, 256, 256, 40), (8, 1, 512, 256, 300)])
def test_sigmoid_moe_on_grouped_mfma_gemms(E, k, F, W, T):
    """Shapes the framework's grouped MFMA expert GEMMs tile: rows scaled by their score, then the
    interleaved gate|up GEMM with the SiLU epilogue and the down GEMM, against the fp32 composition."""
    from polykey_service_amd.ops import gemm
    dev = torch.device("cuda")
    assert moe.mfma_experts_ok(E, F, W, torch.bfloat16, dev)
    x = torch.randn(T, W)
    rw = torch.randn(E, W) * 0.3
    ids, wts = moe.route_sigmoid_topk(x, rw, k)
    gate, up, down = ((torch.randn(E, F, W) * 0.1).bfloat16(), (torch.randn(E, F, W) * 0.1).bfloat16(),
                      (torch.randn(E, W, F) * 0.1).bfloat16())
    want = moe.input_scaled_moe(x, x.bfloat16(), ids, wts, gate, up, down)
    w13 = torch.stack([gemm.interleave_gate_up(gate[e], up[e]) for e in range(E)]).to(dev)
    w2 = down.to(dev)
    for packed in (False, True):
        w13_p = gemm.pack_weight(w13.view(E * 2 * F, W)).view(E, 2 * F, W) if packed else None
        w2_p = gemm.pack_weight(w2.view(E * W, F)).view(E, W, F) if packed else None
        got = moe.input_scaled_moe(x.to(dev), x.bfloat16().to(dev), ids.to(dev), wts.to(dev), None, None, None, w13, w2,
                                   w13_p, w2_p)
        err = (got.cpu() - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()
        assert float(err) < 1e-2, float(err)  # bf16 rounding of the scaled rows, h and y
        assert float((got.cpu() - want).abs().max()) < 0.05 * float(want.abs().max())


@pytest.mark.parametrize("dt", DTYPES)
def test_sum_gain_norm_fused_combine_and_state_save(dt):
    dev = torch.device("cuda")
    T, W, top = 9, 72, 2
    x, yrows = torch.randn(T, W), torch.randn(T * top + 3, W).to(dt)
    inv = torch.randperm(T * top + 3)[:T * top].to(torch.int32)
    inv[5] = -1
    g = torch.tensor([0.9])
    m = batch_meta([4, 1, 4], [4, 20, 9], 4, torch.device("cpu"))
    sl = torch.tensor([2, -1, 0], dtype=torch.int32)
    st_c, st_g = torch.randn(3, W), None
    st_g = st_c.to(dev)
    w_out, w_act = stream.sum_gain_norm(x, yrows, 2.0, g, 1e-5, out=torch.zeros(T, W), act_dtype=dt, gather=(inv, top),
                                        save=(st_c, m["tseq"], m["cu_q"], sl))
    g_out, g_act = stream.sum_gain_norm(x.to(dev), yrows.to(dev), 2.0, g.to(dev), 1e-5, out=torch.zeros(T, W, device=dev),
                                        act_dtype=dt, gather=(inv.to(dev), top),
                                        save=(st_g, m["tseq"].to(dev), m["cu_q"].to(dev), sl.to(dev)))
    torch.testing.assert_close(g_out.cpu(), w_out, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(g_act.cpu().float(), w_act.float(), **tol(dt))
    torch.testing.assert_close(st_g.cpu(), st_c)
    assert torch.equal(st_c[2], x[3]) and torch.equal(st_c[0], x[8])
