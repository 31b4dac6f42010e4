"""HIP sequence-state kernels against the torch reference ops (the same
functions on CPU tensors), fp32 and bf16, over a packed step with a decode
run, a fresh prompt portion, a continuing portion and a slot-less pad run."""
import pytest
import torch

from kubeai_amd.ops import seq as sops

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


RUNS = "short"


def _meta(device, block_tables=None):
    # (length, slot, first position)
    runs = [(1, 2, 37), (1, 0, 5), (19, 3, 0), (7, 1, 30), (2, 5, 64), (5, -1, 0)]
    if RUNS == "long":  # runs that span several scan segments / staging tiles
        runs = [(1, 2, 37), (700, 3, 0), (130, 1, 77), (64, 4, 5), (385, 0, 9), (3, -1, 0)]
    pos = torch.cat([torch.arange(p, p + n) for n, _, p in runs]).int()
    return sops.SeqMeta.build([(n, s) for n, s, _ in runs], pos.to(device), device,
                              block_tables=block_tables), int(pos.numel())


def _tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def _both(fn, dtype, tensors, states):
    """Run fn on CPU and GPU copies; returns (cpu_out, gpu_out, cpu_states, gpu_states)."""
    outs = []
    for dev in ("cpu", "cuda"):
        t = [x.to(dev) if torch.is_tensor(x) else x for x in tensors]
        st = [x.clone().to(dev) for x in states]
        meta, _ = _meta(dev)
        outs.append((fn(meta, *t, *st), st))
    return outs[0][0], outs[1][0], outs[0][1], outs[1][1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_layernorm(dtype):
    torch.manual_seed(0)
    T, C = 37, 200
    res = torch.randn(T, C) * 3
    br = torch.randn(T, C).to(dtype)
    w, b = torch.randn(C), torch.randn(C)
    want_res = res.clone()
    want = sops.add_layernorm(br, want_res, w, b, 1e-6, dtype)
    got_res = res.cuda()
    got = sops.add_layernorm(br.cuda(), got_res, w.cuda(), b.cuda(), 1e-6, dtype)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))
    torch.testing.assert_close(got_res.cpu(), want_res, atol=1e-6, rtol=1e-6)
    got = sops.add_layernorm(None, res.cuda(), w.cuda(), b.cuda(), 1e-6, dtype)
    want = sops.add_layernorm(None, res.clone(), w, b, 1e-6, dtype)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("groups,act", [(1, "sigmoid"), (5, "silu"), (2, "none")])
def test_gated_rmsnorm(dtype, groups, act):
    torch.manual_seed(1)
    T, C = 23, 160
    o, w = torch.randn(T, C), torch.randn(C)
    wide = torch.randn(T, C + 40).to(dtype)
    gate = wide[:, 40:]
    outw_c = torch.zeros(T, C + 24, dtype=dtype)
    outw_g = outw_c.cuda()
    sops.gated_rmsnorm(o, w, gate, groups, act, 1e-6, outw_c[:, 24:], 1.3)
    sops.gated_rmsnorm(o.cuda(), w.cuda(), wide.cuda()[:, 40:], groups, act, 1e-6,
                       outw_g[:, 24:], 1.3)
    torch.testing.assert_close(outw_g.cpu().float(), outw_c.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols", [70, 71 * 8])
def test_relu_squared(dtype, cols):
    x = torch.randn(33, cols).to(dtype)
    torch.testing.assert_close(sops.relu_squared(x.cuda()).cpu().float(),
                               sops.relu_squared(x).float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,residual", [(4, True), (3, False), (2, False), (7, True)])
@pytest.mark.parametrize("C", [72, 70])
def test_causal_conv(dtype, taps, residual, C):
    torch.manual_seed(2)
    _, T = _meta("cpu")
    wide = torch.randn(T, C + 8).to(dtype)
    w = torch.randn(C, taps)
    tails = torch.randn(6, taps - 1, C)

    def fn(meta, wide, w, tails):
        return sops.causal_conv(wide[:, 8:], w, tails, meta, residual)

    c, g, cs, gs = _both(fn, dtype, [wide, w], [tails])
    torch.testing.assert_close(g.cpu().float(), c.float(), **_tol(dtype))
    torch.testing.assert_close(gs[0].cpu(), cs[0], atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift_mix(dtype):
    torch.manual_seed(3)
    _, T = _meta("cpu")
    C = 96
    h = torch.randn(T, C).to(dtype)
    mu = torch.rand(5, C)
    prev = torch.randn(6, 1, C)
    fn = lambda meta, h, mu, prev: sops.token_shift_mix(h, mu, prev, meta)
    c, g, cs, gs = _both(fn, dtype, [h, mu], [prev])
    torch.testing.assert_close(g.cpu().float(), c.float(), **_tol(dtype))
    torch.testing.assert_close(gs[0].cpu(), cs[0], atol=1e-6, rtol=1e-6)


@pytest.fixture(params=["short", "long"])
def runs(request):
    global RUNS
    RUNS = request.param
    yield request.param
    RUNS = "short"


@pytest.mark.parametrize("dtype", DTYPES)
def test_mingru_scan(dtype, runs):
    torch.manual_seed(4)
    _, T = _meta("cpu")
    n = 300
    zxg = (torch.randn(T, 3 * n) * 2).to(dtype)
    bz, bx = torch.randn(n), torch.randn(n)
    st = torch.randn(6, n)
    fn = lambda meta, zxg, bz, bx, st: sops.mingru_scan(zxg, bz, bx, st, meta)
    c, g, cs, gs = _both(fn, dtype, [zxg, bz, bx], [st])
    torch.testing.assert_close(g.cpu().float(), c.float(), **_tol(dtype))
    torch.testing.assert_close(gs[0].cpu(), cs[0], atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(3, 48, 48), (3, 16, 80), (1, 64, 64), (2, 128, 128),
                                    (2, 40, 40)])
def test_linear_attn_scan_per_token_decay(dtype, H, D, Dv, runs):
    if D != Dv:
        pytest.skip("bonus form pairs equal key/value sizes in the model; "
                    "unequal sizes are covered by the constant-decay form")
    torch.manual_seed(5)
    _, T = _meta("cpu")
    wide = torch.randn(T, 3 * H * D + 8).to(dtype)
    dec = (torch.randn(T, H, D) - 2).to(dtype)
    u, w0 = torch.randn(H, D) * 0.5, torch.randn(H * D) * 0.5
    st = torch.randn(6, H, D, Dv)

    def fn(meta, wide, dec, u, w0, st):
        q = wide[:, 8 : 8 + H * D].unflatten(-1, (H, D))
        k = wide[:, 8 + H * D : 8 + 2 * H * D].unflatten(-1, (H, D))
        v = wide[:, 8 + 2 * H * D :].unflatten(-1, (H, Dv))
        return sops.linear_attn_scan(q, k, v, dec, u, st, meta, w_bias=w0)

    c, g, cs, gs = _both(fn, dtype, [wide, dec, u, w0], [st])
    torch.testing.assert_close(g.cpu(), c, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(gs[0].cpu(), cs[0], atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(5, 64, 64), (3, 16, 80), (2, 40, 24), (2, 32, 24),
                                    (1, 112, 130)])
def test_linear_attn_scan_constant_decay(dtype, H, D, Dv, runs):
    torch.manual_seed(6)
    _, T = _meta("cpu")
    q = (torch.randn(T, H, D) * 0.5).to(dtype)
    k = (torch.randn(T, H, D) * 0.5).to(dtype)
    v = torch.randn(T, H, Dv).to(dtype)
    dec = torch.rand(H) * 0.5 + 0.5
    st = torch.randn(6, H, D, Dv)
    fn = lambda meta, q, k, v, dec, st: sops.linear_attn_scan(
        q, k, v, dec, None, st, meta, silu_inputs=True)
    c, g, cs, gs = _both(fn, dtype, [q, k, v, dec], [st])
    torch.testing.assert_close(g.cpu(), c, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(gs[0].cpu(), cs[0], atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,rot,chunk,window,cap",
                         [(6, 2, 48, 80, 32, 16, 0, 30.0), (4, 1, 32, 32, 16, 0, 0, 0.0),
                          (6, 2, 24, 130, 8, 40, 9, 5.0), (2, 2, 64, 64, 64, 0, 11, 0.0)])
@pytest.mark.parametrize("long_runs", [False, True])
def test_rope_cache_and_masked_attention(dtype, H, G, D, Dv, rot, chunk, window, cap,
                                         long_runs):
    torch.manual_seed(7)
    bs, nblk = 16, 60
    runs = [(1, 2, 37), (1, 0, 5), (19, 3, 0), (7, 1, 30), (2, 5, 64), (5, -1, 0)]
    if long_runs:  # several 16-query tiles, chunk edges inside a tile
        runs = [(1, 2, 37), (150, 3, 0), (77, 1, 130), (33, 4, 15), (5, -1, 0)]
    tables = torch.zeros(len(runs), 14, dtype=torch.int32)
    free = list(torch.randperm(nblk - 1).add(1).tolist())
    for i, (n, s, p) in enumerate(runs):
        if s >= 0:
            for b in range((p + n + bs - 1) // bs):
                tables[i, b] = free.pop()
    pos = torch.cat([torch.arange(p, p + n) for n, _, p in runs]).int()
    T = pos.numel()
    slots = []
    for i, (n, s, p) in enumerate(runs):
        for x in range(p, p + n):
            slots.append(-1 if s < 0 else int(tables[i, x // bs]) * bs + x % bs)
    slots = torch.tensor(slots)
    wide = torch.randn(T, H * D + G * D + G * Dv).to(dtype)
    kc0 = torch.randn(nblk, G, bs, D).to(dtype)
    vc0 = torch.randn(nblk, G, bs, Dv).to(dtype)
    inv = (10000.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)).float()
    res = []
    for dev in ("cpu", "cuda"):
        w = wide.clone().to(dev)
        kc, vc = kc0.clone().to(dev), vc0.clone().to(dev)
        meta = sops.SeqMeta.build([(n, s) for n, s, _ in runs], pos.to(dev), dev,
                                  block_tables=tables.to(dev))
        q = w[:, : H * D].unflatten(-1, (H, D))
        k = w[:, H * D : H * D + G * D].unflatten(-1, (G, D))
        v = w[:, H * D + G * D :].unflatten(-1, (G, Dv))
        sops.rope_pairs_and_cache(q, k, v, pos.to(dev), inv.to(dev), kc, vc,
                                  slots.to(dev))
        out = torch.zeros(T, H * Dv + 8, dtype=dtype, device=dev)
        sops.masked_paged_attention(q, kc, vc, meta, 0.2, out[:, 8:].unflatten(-1, (H, Dv)),
                                    softcap=cap, chunk=chunk, window=window,
                                    out_scale=0.8)
        res.append((w.cpu().float(), kc.cpu().float(), vc.cpu().float(), out.cpu().float()))
    n_real = T - 5  # pad rows attend over block 0, whose content is arbitrary but equal
    for a, b in zip(res[0][:3], res[1][:3]):
        torch.testing.assert_close(b, a, **_tol(dtype))
    torch.testing.assert_close(res[1][3][:n_real], res[0][3][:n_real], **_tol(dtype))
