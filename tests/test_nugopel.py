"""Nugopel (window attention with sink / latent attention / routed experts) in
the engine against the plain oracle in nugopel_oracle.py: every mechanism
alone, prompt vs token-by-token decoding, prompt portions down to two tokens,
unequal batches, reuse of freed cache blocks, keys at window / page edges and
far back (planted so that one score stands out), first tokens, long decoding,
other sizes, and greedy generation through the engine's own scheduler. CPU
runs use the torch reference ops; the same cases run on the GPU kernels under
the gpu marker, where the kernels are also compared one by one with the
reference ops.
"""
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import nugopel_oracle as oracle
from kubeai_amd.engine import EngineConfig, LLMEngine, SamplingParams
from kubeai_amd.ops import seq as sops

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
GPU = [pytest.param("cuda", marks=pytest.mark.gpu)]

# wavelengths of base 100 over 8 dims: 6.3, 19.9, 62.8, 198.7 — with these
# constants one is kept, two are interpolated and one is divided
SCALING = {"factor": 3.0, "low": 1.0, "high": 4.0, "original": 64}


def moe(experts=5, top=2, ff=12, shared=9):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


MOE = moe()


def attn(heads=4, kv=2, dim=10, vdim=6, size=9, rot=8, base=100.0, scaling=SCALING,
         scale=0.45, mlp=MOE):
    mx = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
          "mask": {"size": size}}
    if rot:
        mx["rot"] = {"base": base, "dims": rot}
        if scaling:
            mx["rot"]["scaling"] = scaling
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def lat(heads=3, dim=4, vdim=6, rank=10, scale=0.6, kv_from=None, mlp=MOE):
    mx = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx, "mlp": mlp}


def config(layers, width=32, vocab=50, eps=1e-5):
    return {"architecture": "Nugopel", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "layers": layers}


MIXED = config([attn(), lat(), attn(heads=2, kv=1, dim=6, vdim=12, size=20, rot=4),
                lat(heads=2, dim=8, vdim=4, kv_from=1), lat(rank=7, mlp=None)])


def model_dir(tmp_path, cfg, seed=0, W=None):
    d = str(tmp_path / ("m%d" % seed))
    os.makedirs(d, exist_ok=True)
    W = W if W is not None else oracle.random_weights(cfg, seed)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()},
              os.path.join(d, "model.safetensors"))
    return d, oracle.as_float64(W)


def engine(d, device, dtype="float32", blocks=64, seqs=4):
    return LLMEngine(EngineConfig(
        model=d, device=device, dtype=dtype, num_gpu_blocks=blocks,
        max_num_seqs=seqs, max_model_len=1 << 20, max_num_batched_tokens=1 << 20,
        enable_prefix_caching=False, enable_graphs=False))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(2000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got, want):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else got
    return np.abs(got - want).max(-1) / want.std()


def check(got, want, dtype="float32"):
    err = rel_err(got, want).max()
    # bf16: the widths here are tiny, so roundings do not average out; the
    # reference ops on the CPU land at 0.06 - 0.09 for the same models
    assert err < (2e-4 if dtype == "float32" else 0.15), f"relative error {err:.3g}"


def replay(eng, rid, toks, cuts):
    """Feed toks in portions of the given sizes (the last repeats), wanting
    every position; returns [T, vocab]."""
    rows, at, i = [], 0, 0
    while at < len(toks):
        n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
        part = toks[at : at + n]
        at += n
        i += 1
        out = eng.step_fixed([(rid, part, list(range(n)))],
                             [rid] if at == len(toks) else [])
        rows.append(out[0])
    return torch.cat(rows)


# ---------------------------------------------------------------------------
# mechanisms as functions: the product's ops against the oracle's
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("scaling", [None, SCALING,
                                     {"factor": 8.0, "low": 1.0, "high": 4.0,
                                      "original": 8192}])
@pytest.mark.parametrize("dims,base", [(8, 100.0), (64, 500000.0), (2, 10.0)])
def test_rotary_frequencies(scaling, dims, base):
    from kubeai_amd.models.mixers import scaled_rotary_frequencies

    got = scaled_rotary_frequencies(dims, base, scaling).double().numpy()
    want = oracle.rotary_frequencies(dims, base, scaling)
    assert np.abs(got / want - 1).max() < 1e-6


@pytest.mark.parametrize("device", DEVICES)
def test_router_choice_and_weights(device):
    g = torch.Generator().manual_seed(1)
    z = torch.randn(70, 9, generator=g)
    z[3, 2] = z[3, 7] = 5.0  # equal logits: the lower index wins
    for top in (1, 3, 9):
        dense, w, idx = sops.router_topk(z.to(device), top)
        for t in range(z.shape[0]):
            order = np.argsort(-z[t].double().numpy(), kind="stable")[:top]
            assert idx[t].cpu().tolist() == order.tolist()
            e = np.exp(z[t, order].double().numpy())
            assert np.abs(w[t].cpu().double().numpy() - e / e.sum()).max() < 1e-6
            row = np.zeros(9)
            row[order] = e / e.sum()
            assert np.abs(dense[t].cpu().double().numpy() - row).max() < 1e-6


@pytest.mark.parametrize("device", DEVICES)
def test_sandwich_norm_function(device):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 24, generator=g)
    y = torch.randn(5, 24, generator=g) * 3
    wa, wb = torch.randn(24, generator=g) * 0.1, torch.randn(24, generator=g) * 0.1
    res = x.clone().to(device)
    h = sops.sandwich_rmsnorm(y.to(device), (1 + wb).to(device), res, (1 + wa).to(device),
                              1e-3, torch.float32)
    x2 = x.double().numpy() + oracle.norm_one_plus(y.double().numpy(), wb.double().numpy(), 1e-3)
    assert np.abs(res.cpu().double().numpy() - x2).max() < 1e-5
    want = oracle.norm_one_plus(x2, wa.double().numpy(), 1e-3)
    assert np.abs(h.cpu().double().numpy() - want).max() < 1e-5


# ---------------------------------------------------------------------------
# every mechanism alone, in the engine
# ---------------------------------------------------------------------------
SINGLE = {
    "attention_no_ff": config([attn(mlp=None)]),
    "attention": config([attn()]),
    "attention_all_heads_own_kv": config([attn(heads=3, kv=3, dim=8, vdim=8, rot=8)]),
    "attention_one_kv_head_no_scaling": config([attn(heads=4, kv=1, dim=12, vdim=4, rot=4,
                                                     scaling=None, size=7)]),
    "attention_unrotated": config([attn(rot=0)]),
    "attention_window_of_one": config([attn(size=1)]),
    "attention_window_never_reached": config([attn(size=1000)]),
    "latent_no_ff": config([lat(mlp=None)]),
    "latent": config([lat()]),
    "latent_one_head": config([lat(heads=1, dim=16, vdim=3, rank=5)]),
    "latent_shared": config([lat(), lat(heads=2, dim=6, vdim=8, kv_from=0)]),
    "experts_top_one": config([lat(mlp=moe(experts=4, top=1))]),
    "experts_all_chosen": config([lat(mlp=moe(experts=3, top=3))]),
    "experts_no_shared": config([attn(mlp=moe(shared=0))]),
    "one_expert": config([attn(mlp=moe(experts=1, top=1))]),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_whole_prompt(tmp_path, device, name):
    cfg = SINGLE[name]
    d, W = model_dir(tmp_path, cfg, seed=3)
    toks = tokens(37, cfg["vocab"], 1)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [len(toks)]), want)
    check(replay(engine(d, device), "b", toks, [5, 1]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_after_every_layer(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=4)
    toks = tokens(29, MIXED["vocab"], 2)
    layers = []
    oracle.forward(MIXED, W, toks, capture=layers)
    eng = engine(d, device)
    eng.runner.model.capture_layers = []
    replay(eng, "a", toks, [len(toks)])
    got = torch.stack(eng.runner.model.capture_layers)[:, : len(toks)]
    assert got.shape[0] == len(layers)
    for i, want in enumerate(layers):
        check(got[i], want)


# ---------------------------------------------------------------------------
# prompt vs decoding, portions, first tokens
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 5], [7, 1, 1, 4, 1], [16, 1], [11, 13]])
def test_portions_and_token_by_token(tmp_path, device, cuts):
    d, W = model_dir(tmp_path, MIXED, seed=5)
    toks = tokens(45, MIXED["vocab"], 3)
    check(replay(engine(d, device), "a", toks, cuts), oracle.forward(MIXED, W, toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [1, 2, 3])
def test_first_tokens(tmp_path, device, n):
    d, W = model_dir(tmp_path, MIXED, seed=6)
    toks = tokens(n, MIXED["vocab"], 4)
    want = oracle.forward(MIXED, W, toks)
    check(replay(engine(d, device), "a", toks, [n]), want)
    check(replay(engine(d, device), "b", toks, [1]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_window_passes_over_decoded_tokens(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=7)
    toks = tokens(130, MIXED["vocab"], 5)
    check(replay(engine(d, device), "a", toks, [9, 1]), oracle.forward(MIXED, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_routed_path_for_large_steps(tmp_path, device):
    """Steps above the dense-expert threshold gather tokens per expert; both
    paths must agree with the oracle (and so with each other)."""
    from kubeai_amd.models.mixers import RoutedSquaredReluMoE

    cfg = config([lat(mlp=moe(experts=6, top=2)), attn(mlp=moe(experts=3, top=1, shared=0))])
    d, W = model_dir(tmp_path, cfg, seed=8)
    toks = tokens(RoutedSquaredReluMoE.DENSE_MAX_TOKENS + 44, cfg["vocab"], 6)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [len(toks)]), want)
    check(replay(engine(d, device), "b", toks, [100]), want)


# sizes in multiples of 16: bf16 prompt portions take the matrix-core kernel.
# Every expert is chosen, so that no rounding can flip a routing decision.
SIXTEENS = config(
    [attn(heads=4, kv=2, dim=32, vdim=16, size=40, rot=16, scale=0.18,
          mlp=moe(experts=3, top=3, ff=32, shared=16)),
     lat(heads=2, dim=16, vdim=32, rank=48, scale=0.25, mlp=moe(experts=2, top=2, ff=32)),
     lat(heads=4, dim=8, vdim=16, rank=48, scale=0.3, kv_from=1, mlp=None)],
    width=64, vocab=80)
ODD = config([attn(mlp=moe(experts=3, top=3)), lat(mlp=moe(experts=2, top=2)),
              lat(kv_from=1, mlp=None)])


@pytest.mark.parametrize("device", GPU)
@pytest.mark.parametrize("cfg", [ODD, SIXTEENS], ids=["odd_sizes", "sixteens"])
def test_bfloat16_serving_precision(tmp_path, device, cfg):
    d, W = model_dir(tmp_path, cfg, seed=9)
    toks = tokens(120, cfg["vocab"], 7)
    want = oracle.forward(cfg, W, toks)
    got = replay(engine(d, device, dtype="bfloat16"), "a", toks, [50, 17, 2, 1])
    check(got, want, dtype="bfloat16")
    check(replay(engine(d, device, dtype="float32"), "b", toks, [50, 17, 2, 1]), want)


@pytest.mark.parametrize("device", GPU)
def test_bfloat16_with_routing(tmp_path, device):
    """With a real choice among experts a rounding may flip a close call at a
    position; all but a few positions must still agree."""
    d, W = model_dir(tmp_path, MIXED, seed=10)
    toks = tokens(150, MIXED["vocab"], 8)
    want = oracle.forward(MIXED, W, toks)
    got = replay(engine(d, device, dtype="bfloat16"), "a", toks, [64, 5, 1])
    err = rel_err(got, want)
    assert np.median(err) < 6e-2 and (err < 0.15).mean() > 0.75


# ---------------------------------------------------------------------------
# batches, reuse of blocks
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_matches_each_alone(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=11)
    lens = {"a": 41, "b": 3, "c": 18, "d": 1}
    toks = {r: tokens(n, MIXED["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    want = {r: oracle.forward(MIXED, W, t) for r, t in toks.items()}
    eng = engine(d, device)
    at = {r: 0 for r in toks}
    got = {r: [] for r in toks}
    plan = {"a": [5, 1, 1, 9, 2], "b": [1], "c": [2, 7, 1], "d": [1]}
    step = 0
    while any(at[r] < lens[r] for r in toks):
        entries, end = [], []
        for r in toks:
            if at[r] >= lens[r] or (r == "c" and step % 3 == 1):  # c sits some steps out
                continue
            n = min(plan[r][min(step, len(plan[r]) - 1)], lens[r] - at[r])
            entries.append((r, toks[r][at[r] : at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == lens[r]:
                end.append(r)
        for (r, _, _), rows in zip(entries, eng.step_fixed(entries, end)):
            got[r].append(rows)
        step += 1
    for r in toks:
        check(torch.cat(got[r]), want[r])
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_are_reused(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=12)
    eng = engine(d, device, blocks=5, seqs=2)  # 80 tokens, two sequences
    for i in range(4):
        ta, tb = tokens(40 + i, MIXED["vocab"], 20 + i), tokens(17, MIXED["vocab"], 40 + i)
        ra, rb = "a%d" % i, "b%d" % i
        out = eng.step_fixed([(ra, ta[:30], list(range(30))), (rb, tb[:2], [0, 1])])
        ga, gb = [out[0]], [out[1]]
        out = eng.step_fixed([(rb, tb[2:], list(range(15))), (ra, ta[30:31], [0])], [rb])
        gb.append(out[0])
        ga.append(out[1])
        out = eng.step_fixed([(ra, ta[31:], list(range(len(ta) - 31)))], [ra])
        ga.append(out[0])
        check(torch.cat(ga), oracle.forward(MIXED, W, ta))
        check(torch.cat(gb), oracle.forward(MIXED, W, tb))
    with pytest.raises(Exception):
        eng.step_fixed([("x", tokens(81, MIXED["vocab"], 0), [])])


# ---------------------------------------------------------------------------
# keys at edges: one score made to stand out
# ---------------------------------------------------------------------------
def _planted(device, q_pos, key_pos, window, sink, block=16, decode=False, dtype=torch.float32,
             dims=(2, 1, 8, 4), boost=40.0):
    """Attention output at q_pos when only key_pos carries a large aligned
    key and a marked value: ~marker if visible, ~0 otherwise (with a sink;
    without one an invisible key leaves the plain average of zero values)."""
    H, G, D, Dv = dims
    T = q_pos + 1
    q = torch.zeros(T, H, D)
    k = torch.zeros(T, G, D)
    v = torch.zeros(T, G, Dv)
    q[:, :, 0] = 1.0
    k[key_pos, :, 0] = boost
    v[key_pos, :, :] = 7.0
    pos = np.arange(T)
    vis = (pos[None, :] <= pos[:, None])
    if window:
        vis &= (pos[:, None] - pos[None, :]) < window
    s = q[:, 0].double().numpy() @ k[:, 0].double().numpy().T
    want = (oracle.softmax_visible(s, vis, sink) @ v[:, 0].double().numpy())[q_pos]
    nblk = (T + block - 1) // block
    perm = torch.randperm(nblk + 3, generator=torch.Generator().manual_seed(T)).tolist()
    table = torch.tensor([perm[:nblk]], dtype=torch.int32)
    kc = torch.zeros(nblk + 3, G, block, D)
    vc = torch.zeros(nblk + 3, G, block, Dv)
    tp = torch.arange(T)
    kc[table[0][tp // block].long(), :, tp % block] = k
    vc[table[0][tp // block].long(), :, tp % block] = v
    if decode:
        runs, positions, qq = [(1, 0)], torch.tensor([q_pos], dtype=torch.int32), q[q_pos:]
    else:
        lo = max(0, q_pos - 20)
        runs, positions = [(q_pos + 1 - lo, 0)], torch.arange(lo, q_pos + 1, dtype=torch.int32)
        qq = q[lo:]
    meta = sops.SeqMeta.build(runs, positions.to(device), device,
                              block_tables=table.to(device))
    out = torch.zeros(qq.shape[0], H, Dv, device=device, dtype=dtype)
    sops.masked_paged_attention(qq.to(device, dtype).contiguous(), kc.to(device, dtype),
                                vc.to(device, dtype), meta, 1.0, out, window=window,
                                sink=sink)
    return out[-1].float().cpu().double().numpy(), want


EDGES = [
    (10, 99, 90, True),     # last key the window keeps
    (10, 99, 89, False),    # first key it has dropped
    (16, 47, 32, True),     # window edge on a page border
    (16, 47, 31, False),
    (16, 48, 33, True),
    (16, 48, 32, False),
    (1, 30, 30, True),      # a window of one sees itself only
    (1, 30, 29, False),
    (150, 500, 351, True),
    (150, 500, 350, False),
    (0, 700, 3, True),      # no window: a key hundreds of tokens back
    (0, 1029, 0, True),     # the very first key, far back
    (20, 5, 0, True),       # window longer than the sequence
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("window,q_pos,key_pos,visible", EDGES)
def test_planted_key_at_edges(device, decode, window, q_pos, key_pos, visible):
    got, want = _planted(device, q_pos, key_pos, window, sink=True, decode=decode)
    assert (want[0] > 6.9) == visible
    assert (want[0] < 0.1) == (not visible)
    assert np.abs(got - want[None, :]).max() < 1e-4


@pytest.mark.parametrize("device", GPU)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("window,q_pos,key_pos,visible", EDGES)
def test_planted_key_at_edges_matrix_core_kernel(device, decode, window, q_pos, key_pos,
                                                 visible):
    got, want = _planted(device, q_pos, key_pos, window, sink=True, decode=decode,
                         dtype=torch.bfloat16, dims=(4, 2, 32, 16), boost=32.0)
    assert (want[0] > 6.9) == visible
    assert np.abs(got - want[None, :]).max() < 0.05


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("boost", [-30.0, 0.0, 2.0])
def test_sink_takes_its_share(device, boost):
    """Scores far below zero leave almost everything to the sink (output near
    zero); at score 0 over n keys the values get n / (n + 1)."""
    for decode in (False, True):
        got, want = _planted(device, 12, 12, 1, sink=True, decode=decode, boost=boost)
        assert np.abs(got - want[None, :]).max() < 1e-5
        share = np.exp(boost) / (1 + np.exp(boost))
        assert abs(want[0] - 7.0 * share) < 1e-9
        got, want = _planted(device, 12, 12, 1, sink=False, decode=decode, boost=boost)
        assert abs(want[0] - 7.0) < 1e-9 and np.abs(got - 7.0).max() < 1e-5


@pytest.mark.parametrize("device", DEVICES)
def test_window_edge_through_the_model(tmp_path, device):
    """One window-attention layer: the logits at i depend on the token at
    i - size + 1 and not on the one at i - size, in a prompt and decoded."""
    size = 9
    cfg = config([attn(size=size, mlp=None)])
    d, W = model_dir(tmp_path, cfg, seed=13)
    a = tokens(40, cfg["vocab"], 30)
    i = 33
    inside, outside = list(a), list(a)
    inside[i - size + 1] = (a[i - size + 1] + 1) % cfg["vocab"]
    outside[i - size] = (a[i - size] + 1) % cfg["vocab"]
    wa = oracle.forward(cfg, W, a)[i]
    w_in = oracle.forward(cfg, W, inside)[i]
    assert np.abs(w_in - wa).max() > 1e-3
    for n, cuts in enumerate([[40], [20, 1]]):
        eng = engine(d, device)
        ga = replay(eng, "a%d" % n, a, cuts)[i].double().cpu().numpy()
        gi = replay(eng, "i%d" % n, inside, cuts)[i].double().cpu().numpy()
        go = replay(eng, "o%d" % n, outside, cuts)[i].double().cpu().numpy()
        assert np.abs(go - ga).max() < 1e-5 * wa.std()
        assert np.abs((gi - ga) - (w_in - wa)).max() < 2e-4 * wa.std()


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_reaches_logits_through_latents(tmp_path, device):
    """A latent layer that reads another's cache sees every earlier token:
    changing token 2 changes logits 300 tokens later as the oracle says."""
    cfg = config([attn(size=4), lat(scale=2.0), lat(kv_from=1, scale=2.0)])
    d, W = model_dir(tmp_path, cfg, seed=14)
    a = tokens(300, cfg["vocab"], 31)
    b = list(a)
    b[2] = (a[2] + 1) % cfg["vocab"]
    eng = engine(d, device)
    ga = replay(eng, "a", a, [250, 3, 1])[-1].double().cpu().numpy()
    gb = replay(eng, "b", b, [250, 3, 1])[-1].double().cpu().numpy()
    wa, wb = oracle.forward(cfg, W, a)[-1], oracle.forward(cfg, W, b)[-1]
    assert np.abs(wa - wb).max() > 1e-5 * wa.std()
    assert np.abs((ga - gb) - (wa - wb)).max() / wa.std() < 2e-4


# ---------------------------------------------------------------------------
# other sizes and orders
# ---------------------------------------------------------------------------
OTHER = {
    "latent_first_then_shared_twice": config(
        [lat(heads=5, dim=6, vdim=2, rank=12), lat(heads=1, dim=2, vdim=20, rank=12, kv_from=0),
         attn(heads=6, kv=3, dim=4, vdim=20, size=5, rot=2),
         lat(heads=2, dim=6, vdim=6, rank=12, kv_from=0)], width=24, vocab=33),
    "two_latents_of_their_own": config(
        [lat(rank=6), lat(rank=20, heads=2, dim=10, vdim=10), lat(rank=6, kv_from=0),
         lat(rank=20, kv_from=1)], width=40, vocab=70, eps=1e-3),
    "rotation_over_the_whole_head": config(
        [attn(heads=2, kv=2, dim=6, vdim=6, rot=6, base=7.0, scale=1.3,
              scaling={"factor": 2.0, "low": 0.5, "high": 3.0, "original": 20}),
         attn(heads=8, kv=2, dim=4, vdim=2, rot=2, size=33)], width=16),
    "wide_experts": config([attn(mlp=moe(experts=7, top=5, ff=30, shared=3)),
                            lat(mlp=moe(experts=2, top=1, ff=50, shared=40))], width=48),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(tmp_path, device, name):
    cfg = OTHER[name]
    d, W = model_dir(tmp_path, cfg, seed=15)
    toks = tokens(53, cfg["vocab"], 9)
    check(replay(engine(d, device), "a", toks, [19, 2, 6, 1]), oracle.forward(cfg, W, toks))


def test_unconsumed_tensor_is_an_error(tmp_path):
    cfg = config([lat()])
    W = oracle.random_weights(cfg, 16)
    W["l0.mix.extra"] = torch.zeros(3).bfloat16()
    d, _ = model_dir(tmp_path, cfg, seed=16, W=W)
    with pytest.raises(ValueError):
        engine(d, "cpu")


def test_token_ids_outside_the_vocabulary_are_rejected(tmp_path):
    cfg = config([lat(mlp=None)])
    d, _ = model_dir(tmp_path, cfg, seed=21)
    eng = engine(d, "cpu")
    with pytest.raises(ValueError):
        eng.step_fixed([("a", [1, cfg["vocab"]], [0])])
    with pytest.raises(ValueError):
        eng.add_request([3, -1])
    assert eng.step_fixed([("b", [1, cfg["vocab"] - 1], [1])], ["b"])[0].shape[0] == 1


def test_latent_source_must_cache_a_latent(tmp_path):
    cfg = config([attn(), lat(kv_from=0)])
    d, _ = model_dir(tmp_path, cfg, seed=17, W={"embed": torch.zeros(1).bfloat16()})
    with pytest.raises(ValueError):
        engine(d, "cpu")


# ---------------------------------------------------------------------------
# generation through the engine's own entry point and scheduler
# ---------------------------------------------------------------------------
def _generate(eng, prompts, max_tokens, arrive_every=0):
    pending = list(prompts.items())
    if not arrive_every:
        for rid, t in pending:
            eng.add_request(t, SamplingParams(max_tokens=max_tokens, ignore_eos=True),
                            request_id=rid)
        pending = []
    done, steps = {}, 0
    while (pending or eng.has_work()) and steps < 600:
        if pending and steps % arrive_every == 0:
            rid, t = pending.pop(0)
            eng.add_request(t, SamplingParams(max_tokens=max_tokens, ignore_eos=True),
                            request_id=rid)
        for o in eng.step():
            if o.finished:
                done[o.request_id] = list(o.output_token_ids)
        steps += 1
    return done


def _assert_greedy(cfg, W, prompts, done, tol):
    assert set(done) == set(prompts)
    for rid, t in prompts.items():
        gen = done[rid]
        logits = oracle.forward(cfg, W, t + gen)
        for i, tok in enumerate(gen):
            row = logits[len(t) - 1 + i]
            assert row[tok] >= row.max() - tol * row.std(), (rid, i)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("prefix_caching", [False, True])
def test_greedy_generation_through_scheduler(tmp_path, device, prefix_caching):
    d, W = model_dir(tmp_path, MIXED, seed=18)
    eng = LLMEngine(EngineConfig(
        model=d, device=device, dtype="float32", num_gpu_blocks=40, max_num_seqs=3,
        max_model_len=256, max_num_batched_tokens=24,  # prompts get chunked
        enable_prefix_caching=prefix_caching, enable_graphs=False))
    common = tokens(36, MIXED["vocab"], 49)  # shared by two prompts: cached blocks
    prompts = {"p%d" % i: tokens(n, MIXED["vocab"], 50 + i)
               for i, n in enumerate([31, 5, 47, 12, 2])}
    prompts["c0"] = common + tokens(7, MIXED["vocab"], 60)
    prompts["c1"] = common + tokens(3, MIXED["vocab"], 61)
    done = _generate(eng, prompts, 12)
    assert all(len(g) == 12 for g in done.values())
    _assert_greedy(MIXED, W, prompts, done, 1e-3)
    if prefix_caching:
        assert eng.block_manager.cache_hit_tokens > 0
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


def test_preemption_and_abort_keep_the_cache_consistent(tmp_path):
    d, W = model_dir(tmp_path, MIXED, seed=19)
    eng = LLMEngine(EngineConfig(
        model=d, device="cpu", dtype="float32", num_gpu_blocks=6, max_num_seqs=3,
        max_model_len=128, max_num_batched_tokens=64))  # tight pool: preemption
    prompts = {"q%d" % i: tokens(30, MIXED["vocab"], 70 + i) for i in range(3)}
    for rid, t in prompts.items():
        eng.add_request(t, SamplingParams(max_tokens=20, ignore_eos=True), request_id=rid)
    done, steps = {}, 0
    while eng.has_work() and steps < 600:
        if steps == 3:
            eng.abort_request("q1")
        for o in eng.step():
            if o.finished:
                done[o.request_id] = list(o.output_token_ids)
        steps += 1
    _assert_greedy(MIXED, W, {r: prompts[r] for r in ("q0", "q2")},
                   {r: done[r] for r in ("q0", "q2")}, 1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graph_replays_match_oracle(tmp_path, dtype):
    """Pure-decode steps replay a captured graph; prompt portions of later
    arrivals run eagerly between replays. Every generated token is checked."""
    cfg = MIXED if dtype == "float32" else SIXTEENS
    d, W = model_dir(tmp_path, cfg, seed=20)
    eng = LLMEngine(EngineConfig(
        model=d, device="cuda", dtype=dtype, num_gpu_blocks=64, max_num_seqs=6,
        max_model_len=512, max_num_batched_tokens=64, enable_graphs=True))
    prompts = {"g%d" % i: tokens(n, cfg["vocab"], 90 + i)
               for i, n in enumerate([9, 33, 4, 70, 18, 2, 25])}
    done = _generate(eng, prompts, 24, arrive_every=5)
    assert eng.runner._graphs, "no decode graph was captured"
    _assert_greedy(cfg, W, prompts, done, 1e-3 if dtype == "float32" else 0.25)


def test_served_over_http_with_sampling():
    """The family behind the engine's OpenAI server: greedy and sampled
    completions through the same scheduler, sampler and tokenizer plumbing."""
    from fastapi.testclient import TestClient

    from kubeai_amd.engine.server import EngineServer, build_app

    cfg = EngineConfig(model="nugopel-tiny", device="cpu", num_gpu_blocks=64,
                       max_model_len=256, max_num_seqs=4)
    server = EngineServer(cfg, "latent")
    server.start()
    server._ready.wait(timeout=60)
    try:
        with TestClient(build_app(server)) as c:
            body = {"model": "latent", "prompt": "a b c d e", "max_tokens": 6,
                    "temperature": 0}
            r = c.post("/v1/completions", json=body)
            assert r.status_code == 200, r.text
            greedy = r.json()
            assert greedy["usage"]["completion_tokens"] >= 1
            r2 = c.post("/v1/completions", json=body)
            assert r2.json()["choices"][0]["text"] == greedy["choices"][0]["text"]
            r3 = c.post("/v1/completions", json=dict(body, temperature=0.9, top_p=0.9,
                                                     seed=3))
            assert r3.status_code == 200, r3.text
    finally:
        server.stop()


# ---------------------------------------------------------------------------
# the kernels one by one against the reference ops
# ---------------------------------------------------------------------------
def _both(fn, *args):
    """Run an op on CPU copies and on GPU copies of the tensor arguments;
    returns the two argument lists (in-place results) and return values."""
    cpu = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
    gpu = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    return cpu, fn(*cpu), gpu, fn(*gpu)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [24, 256, 1000])
def test_kernel_sandwich_norm(dtype, C):
    g = torch.Generator().manual_seed(C)
    for branch_dtype in (dtype, torch.float32):
        y = (torch.randn(7, C, generator=g) * 2).to(branch_dtype)
        x = torch.randn(7, C, generator=g)
        wa, wb = 1 + 0.1 * torch.randn(C, generator=g), 1 + 0.1 * torch.randn(C, generator=g)
        cpu, hc, gpu, hg = _both(
            lambda y, wb, x, wa: sops.sandwich_rmsnorm(y, wb, x, wa, 1e-5, dtype), y, wb, x, wa)
        assert (cpu[2] - gpu[2].cpu()).abs().max() < 1e-5
        assert (hc.float() - hg.cpu().float()).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)
    cpu, hc, gpu, hg = _both(
        lambda x, wa: sops.sandwich_rmsnorm(None, None, x, wa, 1e-5, dtype), x, wa)
    assert (hc.float() - hg.cpu().float()).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,half", [(4, 2, 10, 6, 4), (6, 3, 80, 40, 20), (3, 1, 16, 8, 8),
                                           (2, 2, 8, 8, 0)])
def test_kernel_qknorm_rotary_cache(dtype, H, G, D, Dv, half):
    g = torch.Generator().manual_seed(H * D)
    T, bs, nb = 21, 16, 5
    qkv = torch.randn(T, (H + G) * D + G * Dv, generator=g).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(H * D, generator=g), 1 + 0.2 * torch.randn(G * D, generator=g)
    pos = torch.randint(0, 3000, (T,), generator=g).int()
    inv = torch.rand(half, generator=g)
    slots = torch.randperm(nb * bs, generator=g)[:T]
    slots[5] = -1
    tol = 1e-4 if dtype == torch.float32 else 6e-2

    def run(qkv, qw, kw, pos, inv, slots):
        kc = torch.zeros(nb, G, bs, D, dtype=dtype, device=qkv.device)
        vc = torch.zeros(nb, G, bs, Dv, dtype=dtype, device=qkv.device)
        q = qkv[:, : H * D].unflatten(-1, (H, D))
        k = qkv[:, H * D : (H + G) * D].unflatten(-1, (G, D))
        v = qkv[:, (H + G) * D :].unflatten(-1, (G, Dv))
        sops.qknorm_rope_half_and_cache(q, k, v, qw, kw, 1e-5, pos, inv, kc, vc, slots)
        return q.float().cpu(), kc.float().cpu(), vc.float().cpu()

    _, c, _, gq = _both(run, qkv, qw, kw, pos, inv, slots)
    for a, b in zip(c, gq):
        assert (a - b).abs().max() < tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernel_latent_cache_gate_and_weighted_activation(dtype):
    g = torch.Generator().manual_seed(5)
    tol = 1e-5 if dtype == torch.float32 else 4e-2
    x = torch.randn(19, 50, generator=g).to(dtype)
    w = 1 + 0.2 * torch.randn(30, generator=g)
    slots = torch.randperm(64, generator=g)[:19]
    slots[0] = -1

    def to_cache(x, w, slots):
        cache = torch.zeros(4, 1, 16, 30, dtype=dtype, device=x.device)
        sops.rmsnorm_to_cache(x[:, 20:], w, 1e-5, cache, slots)
        return cache.float().cpu()

    _, c, _, gg = _both(to_cache, x, w, slots)
    assert (c - gg).abs().max() < tol
    _, c, _, gg = _both(lambda x: sops.sigmoid_gate(x[:, :20].contiguous(), x[:, 30:]), x)
    assert (c.float() - gg.cpu().float()).abs().max() < tol
    u = torch.randn(19, 5 * 8 + 3, generator=g).to(dtype)
    rw = torch.rand(19, 5, generator=g)
    _, c, _, gg = _both(lambda u, rw: sops.relu_squared_weighted(u, rw, 8), u, rw)
    assert (c.float() - gg.cpu().float()).abs().max() < tol * 4
    _, c, _, gg = _both(lambda u, rw: sops.relu_squared_weighted(u, rw[:, 2:3], 43), u, rw)
    assert (c.float() - gg.cpu().float()).abs().max() < tol * 4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,shared", [(4, 2, 10, 6, False), (8, 2, 32, 16, False),
                                             (3, 1, 48, 48, True), (2, 1, 20, 20, True),
                                             (2, 1, 192, 192, True)])
def test_kernel_attention_with_sink_and_window(dtype, H, G, D, Dv, shared):
    """Random runs (decode tokens beside prompt portions) over shuffled pages,
    with and without sink and window; shared = keys and values are one cache
    (latent attention)."""
    g = torch.Generator().manual_seed(H * D + Dv)
    bs, lens, news = 16, [70, 1, 33, 150], [1, 1, 20, 64]
    nb = sum((n + bs - 1) // bs for n in lens) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    kc = (torch.randn(nb, G, bs, D, generator=g) * 0.5).to(dtype)
    vc = kc if shared else torch.randn(nb, G, bs, Dv, generator=g).to(dtype)
    tables, runs, positions, at = [], [], [], 0
    for n, new in zip(lens, news):
        k = (n + bs - 1) // bs
        tables.append(perm[at : at + k] + [0] * (10 - k))
        at += k
        runs.append((new, -1))
        positions += list(range(n - new, n))
    T = len(positions)
    q = torch.randn(T, H, D, generator=g).to(dtype)
    tol = 1e-4 if dtype == torch.float32 else 5e-2
    for window, sink in [(0, False), (0, True), (24, True), (7, False)]:
        outs = []
        for dev in ("cpu", "cuda"):
            meta = sops.SeqMeta.build(runs, torch.tensor(positions, dtype=torch.int32).to(dev),
                                      dev, block_tables=torch.tensor(tables, dtype=torch.int32).to(dev))
            out = torch.zeros(T, H, Dv, dtype=dtype, device=dev)
            kcd = kc.to(dev)
            sops.masked_paged_attention(q.to(dev), kcd, kcd if shared else vc.to(dev), meta,
                                        D ** -0.5, out, window=window, sink=sink)
            outs.append(out.float().cpu())
        assert (outs[0] - outs[1]).abs().max() < tol, (window, sink)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,A,B", [(1, 1, 16, 16), (37, 3, 32, 48), (70, 2, 192, 16),
                                     (5, 4, 10, 6), (130, 2, 128, 128)])
def test_kernel_head_linear(dtype, T, H, A, B):
    g = torch.Generator().manual_seed(T + A)
    wide = torch.randn(T, H * A + 8, generator=g).to(dtype)  # x is a column view
    w = (torch.randn(H, B, A, generator=g) * A ** -0.5).to(dtype)
    gate = torch.randn(T, H * B + 8, generator=g).to(dtype)
    tol = 1e-4 if dtype == torch.float32 else 5e-2
    for gated in (False, True):
        def run(wide, w, gate):
            x = wide[:, 8:].unflatten(-1, (H, A))
            return sops.head_linear(x, w, gate[:, : H * B] if gated else None)

        _, c, _, gg = _both(run, wide, w, gate)
        assert (c.float() - gg.cpu().float()).abs().max() < tol


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,shared", [(16, 1, 128, 128, True), (16, 2, 32, 16, False),
                                             (20, 1, 48, 48, True), (4, 4, 64, 64, False),
                                             (9, 1, 16, 128, False)])
def test_kernel_decode_attention_grouped_heads(H, G, D, Dv, shared):
    """Pure decode steps in bf16 with eight or more heads per key/value head
    take the kernel whose tile rows are the heads of a group (keys split over
    blocks, joined by a second kernel); contexts around the 32-key tile and
    the split borders, with and without window and sink."""
    g = torch.Generator().manual_seed(H + D)
    bs, lens = 16, [1, 31, 32, 33, 127, 128, 129, 200, 1000]
    nb = sum((n + bs - 1) // bs for n in lens) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    kc = (torch.randn(nb, G, bs, D, generator=g) * 0.5).bfloat16()
    vc = kc if shared else torch.randn(nb, G, bs, Dv, generator=g).bfloat16()
    width = max((n + bs - 1) // bs for n in lens)
    tables, at = [], 0
    for n in lens:
        k = (n + bs - 1) // bs
        tables.append(perm[at : at + k] + [0] * (width - k))
        at += k
    runs = [(1, -1)] * len(lens)
    positions = [n - 1 for n in lens]
    q = torch.randn(len(lens), H, D, generator=g).bfloat16()
    for window, sink in [(0, False), (0, True), (40, True), (1, False)]:
        outs = []
        for dev in ("cpu", "cuda"):
            meta = sops.SeqMeta.build(runs, torch.tensor(positions, dtype=torch.int32).to(dev),
                                      dev, block_tables=torch.tensor(tables, dtype=torch.int32).to(dev))
            out = torch.zeros(len(lens), H, Dv, dtype=torch.bfloat16, device=dev)
            kcd = kc.to(dev)
            sops.masked_paged_attention(q.to(dev), kcd, kcd if shared else vc.to(dev), meta,
                                        D ** -0.5, out, window=window, sink=sink)
            outs.append(out.float().cpu())
        assert (outs[0] - outs[1]).abs().max() < 5e-2, (window, sink)
