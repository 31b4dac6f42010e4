"""Dulotar (hybrid recurrent / chunked-attention decoder) in the engine against
the plain oracle in dulotar_oracle.py: every mixer alone, prompt vs
token-by-token decoding, prompt portions down to two tokens, unequal batches,
reuse of freed cache blocks and state slots, keys at chunk / page edges and
far back, first tokens, long decoding, other sizes, and greedy generation
through the engine's own scheduler. CPU runs use the torch reference ops; the
same cases run on the GPU kernels under the gpu marker.
"""
import copy
import json
import os

import pytest
import torch
from safetensors.torch import save_file

import dulotar_oracle as oracle
from kubeai_amd.engine import EngineConfig, LLMEngine, SamplingParams
from kubeai_amd.ops import seq as sops

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def left(heads=4, kv=2, dim=8, vdim=12, conv=3, size=10, rot=8, base=100.0,
         scale=0.4, cap=6.0):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv,
            "mask": {"size": size}, "rot": {"base": base, "dims": rot},
            "scale": scale, "softcap": cap}


def right(heads=3, dim=4, vdim=10, decay=(0.5, 0.9, 0.97)):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def par(l=None, r=None, ls=0.7, rs=1.2, mlp=None):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": l or left(), "right": r or right(),
                      "left_scale": ls, "right_scale": rs}}


def gru(n=24, mlp=None):
    return {"type": "mingru", "mixer": {"width": n}, "mlp": mlp}


def wkv(heads=3, dim=8, mlp=None):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


FF = {"kind": "dense", "ff": 40}


def config(layers, width=32, vocab=50, taps=3, scale=3.0):
    return {"architecture": "Dulotar", "vocab": vocab, "width": width,
            "canon": {"taps": taps}, "embedding": {"scale": scale},
            "norm": {"eps": 1e-5}, "layers": layers}


MIXED = config([wkv(), gru(), par(mlp=FF), dict(gru(), weights_of=1),
                dict(par(mlp=FF), weights_of=2)])


def model_dir(tmp_path, cfg, seed=0, W=None):
    d = str(tmp_path / ("m%d" % seed))
    os.makedirs(d, exist_ok=True)
    W = W if W is not None else oracle.random_weights(cfg, seed)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()},
              os.path.join(d, "model.safetensors"))
    return d, W


def engine(d, device, dtype="float32", blocks=64, seqs=4):
    return LLMEngine(EngineConfig(
        model=d, device=device, dtype=dtype, num_gpu_blocks=blocks,
        max_num_seqs=seqs, max_model_len=1 << 20, max_num_batched_tokens=1 << 20,
        enable_graphs=False))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def check(got, want, dtype="float32"):
    got, want = got.double().cpu(), want.double()
    tol = 2e-4 if dtype == "float32" else 6e-2
    scale = want.std().item()
    err = (got - want).abs().max().item() / scale
    assert err < tol, f"relative error {err:.3g}"


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
# every mechanism alone
# ---------------------------------------------------------------------------
SINGLE = {
    "mingru": config([gru()]),
    "mingru_ff": config([gru(mlp=FF)], taps=2),
    "wkv": config([wkv()]),
    "wkv_one_head": config([wkv(heads=1, dim=16)], taps=5),
    "chunked_only": config([par(rs=0.0)]),
    "lightning_only": config([par(ls=0.0)]),
    "parallel": config([par(mlp=FF)]),
    "full_rotary_no_group": config([par(l=left(heads=3, kv=3, dim=6, vdim=6, rot=6))]),
    "one_kv_head_partial_rotary": config([par(l=left(heads=4, kv=1, dim=12, vdim=4, rot=4,
                                                     conv=2, size=7))]),
    "right_equal_sizes": config([par(r=right(heads=1, dim=8, vdim=8, decay=(0.8,)))]),
    "shared_weights": config([gru(), dict(gru(), weights_of=0), wkv(),
                              dict(wkv(), weights_of=2)]),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mixer_whole_prompt(tmp_path, device, name):
    cfg = SINGLE[name]
    d, W = model_dir(tmp_path, cfg, seed=3)
    toks = tokens(37, cfg["vocab"], 1)
    want = oracle.forward(cfg, W, toks)
    got = replay(engine(d, device), "a", toks, [len(toks)])
    check(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_after_every_layer(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=4)
    toks = tokens(29, MIXED["vocab"], 2)
    _, layers = oracle.forward(MIXED, W, toks, return_layers=True)
    eng = engine(d, device)
    eng.runner.model.capture_layers = []
    replay(eng, "a", toks, [len(toks)])
    got = torch.stack(eng.runner.model.capture_layers)[:, : len(toks)]
    for i in range(layers.shape[0]):
        check(got[i], layers[i])


# ---------------------------------------------------------------------------
# prompt vs decoding, portions, first tokens
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 5], [7, 1, 1, 4, 1], [16, 1], [11, 13]])
def test_portions_and_token_by_token(tmp_path, device, cuts):
    d, W = model_dir(tmp_path, MIXED, seed=5)
    toks = tokens(45, MIXED["vocab"], 3)
    want = oracle.forward(MIXED, W, toks)
    check(replay(engine(d, device), "a", toks, cuts), want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [1, 2, 3, 4])
def test_first_tokens(tmp_path, device, n):
    cfg = config([wkv(), par(l=left(conv=4)), gru()], taps=4)
    d, W = model_dir(tmp_path, cfg, seed=6)
    toks = tokens(n, cfg["vocab"], 4)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [n]), want)
    check(replay(engine(d, device), "b", toks, [1]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=7)
    toks = tokens(230, MIXED["vocab"], 5)
    want = oracle.forward(MIXED, W, toks)
    check(replay(engine(d, device), "a", toks, [9, 1]), want)


# sizes in multiples of 16: bf16 prompt portions take the matrix-core
# attention kernel and the register-state scans
MFMA_SIZED = config(
    [wkv(heads=2, dim=16), gru(n=48, mlp=FF),
     par(l=left(heads=4, kv=2, dim=32, vdim=16, conv=3, size=24, rot=16, scale=0.18),
         r=right(heads=2, dim=16, vdim=32, decay=(0.9, 0.99)), mlp=FF)],
    width=64, vocab=80)


@pytest.mark.parametrize("device", [pytest.param("cuda", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("cfg", [MIXED, MFMA_SIZED], ids=["odd_sizes", "sixteens"])
def test_bfloat16_serving_precision(tmp_path, device, cfg):
    d, W = model_dir(tmp_path, cfg, seed=8)
    toks = tokens(120, cfg["vocab"], 6)
    want = oracle.forward(cfg, W, toks)
    got = replay(engine(d, device, dtype="bfloat16"), "a", toks, [50, 17, 2, 1])
    check(got, want, dtype="bfloat16")
    got = replay(engine(d, device, dtype="float32"), "b", toks, [50, 17, 2, 1])
    check(got, want)


# ---------------------------------------------------------------------------
# batches, reuse of blocks and slots
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_matches_each_alone(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=9)
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
    assert eng.state_manager.num_free == 4
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_and_slots_are_reused(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=10)
    eng = engine(d, device, blocks=5, seqs=2)  # 80 tokens, two sequences
    seen_slots = []
    for i in range(5):
        ta, tb = tokens(40 + i, MIXED["vocab"], 20 + i), tokens(17, MIXED["vocab"], 40 + i)
        ra, rb = "a%d" % i, "b%d" % i
        out = eng.step_fixed([(ra, ta[:30], list(range(30))), (rb, tb[:2], [0, 1])])
        seen_slots.append(eng._fixed[ra].state_slot)
        ga, gb = [out[0]], [out[1]]
        out = eng.step_fixed([(rb, tb[2:], list(range(15))), (ra, ta[30:31], [0])], [rb])
        gb.append(out[0])
        ga.append(out[1])
        out = eng.step_fixed([(ra, ta[31:], list(range(len(ta) - 31)))], [ra])
        ga.append(out[0])
        check(torch.cat(ga), oracle.forward(MIXED, W, ta))
        check(torch.cat(gb), oracle.forward(MIXED, W, tb))
    assert len(set(seen_slots)) < len(seen_slots)  # slots came back
    with pytest.raises(Exception):
        eng.step_fixed([("x", tokens(81, MIXED["vocab"], 0), [])])


# ---------------------------------------------------------------------------
# keys at edges: one score made to stand out
# ---------------------------------------------------------------------------
def _planted(device, T, q_pos, key_pos, size, block=16, window=0, decode=False):
    """Attention output at q_pos when only key_pos carries a large aligned
    key and a marked value: ~marker if visible, ~0 otherwise."""
    H, G, D, Dv = 2, 1, 8, 4
    q = torch.zeros(T, H, D)
    k = torch.zeros(T, G, D)
    v = torch.zeros(T, G, Dv)
    q[:, :, 0] = 1.0
    k[key_pos, 0, 0] = 40.0
    v[key_pos, 0, :] = 7.0
    want = oracle.chunk_softmax(q.double(), k.double(), v.double(), 1.0, 1e9,
                                size if size else T + 1)[q_pos]
    nblk = (T + block - 1) // block
    perm = torch.randperm(nblk + 3, generator=torch.Generator().manual_seed(T)).tolist()
    table = torch.tensor([perm[:nblk]], dtype=torch.int32)
    kc = torch.zeros(nblk + 3, G, block, D)
    vc = torch.zeros(nblk + 3, G, block, Dv)
    pos = torch.arange(T)
    kc[table[0][pos // block].long(), :, pos % block] = k
    vc[table[0][pos // block].long(), :, pos % block] = v
    if decode:
        runs, positions, qq = [(1, 0)], torch.tensor([q_pos], dtype=torch.int32), q[q_pos : q_pos + 1]
    else:
        lo = max(0, q_pos - 4)
        runs, positions = [(q_pos + 1 - lo, 0)], torch.arange(lo, q_pos + 1, dtype=torch.int32)
        qq = q[lo : q_pos + 1]
    meta = sops.SeqMeta.build(runs, positions.to(device), device,
                              block_tables=table.to(device))
    out = torch.zeros(qq.shape[0], H, Dv, device=device)
    sops.masked_paged_attention(qq.to(device).contiguous(), kc.to(device), vc.to(device),
                                meta, 1.0, out, chunk=size, window=window)
    return out[-1].cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("size,q_pos,key_pos,visible", [
    (24, 47, 24, True),    # first key of the query's chunk
    (24, 47, 23, False),   # last key of the chunk before
    (24, 48, 47, False),   # query opens a chunk: the previous token is outside
    (24, 48, 48, True),
    (16, 31, 16, True),    # chunk edge on a page border
    (16, 32, 31, False),
    (20, 39, 32, True),    # key at a page border inside the chunk
    (0, 700, 3, True),     # no chunks: a key hundreds of tokens back
    (512, 1000, 512, True),
    (512, 1000, 511, False),
])
def test_planted_key_at_edges(device, decode, size, q_pos, key_pos, visible):
    got, want = _planted(device, q_pos + 1, q_pos, key_pos, size, decode=decode)
    assert (want[0, 0].item() > 6.9) == visible
    assert (got - want).abs().max().item() < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_window_mask_parameter(device):
    # the mask also takes a sliding window (beside or instead of chunks)
    got, _ = _planted(device, 100, 99, 90, 0, window=10)
    assert got[0, 0].item() > 6.9
    got, _ = _planted(device, 100, 99, 89, 0, window=10)
    assert abs(got[0, 0].item()) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_reaches_logits_through_state(tmp_path, device):
    """Changing one early token must change late logits exactly as the oracle
    says (recurrent state carried over many portions and decoded tokens)."""
    cfg = config([gru(), par(l=left(size=8)), wkv()])
    d, W = model_dir(tmp_path, cfg, seed=11)
    a = tokens(150, cfg["vocab"], 30)
    b = list(a)
    b[2] = (a[2] + 1) % cfg["vocab"]
    eng = engine(d, device)
    ga = replay(eng, "a", a, [40, 3, 1])[-1]
    gb = replay(eng, "b", b, [40, 3, 1])[-1]
    wa, wb = oracle.forward(cfg, W, a)[-1], oracle.forward(cfg, W, b)[-1]
    assert (wa - wb).abs().max() > 1e-6  # the oracle itself still remembers
    scale = wa.std().item()
    assert ((ga - gb).double().cpu() - (wa - wb)).abs().max().item() / scale < 2e-4


# ---------------------------------------------------------------------------
# other sizes and orders
# ---------------------------------------------------------------------------
OTHER = {
    "wide_ff_everywhere": config([gru(n=40, mlp=FF), wkv(heads=2, dim=16, mlp=FF),
                                  par(mlp=FF)], width=48, vocab=70, taps=2),
    "attention_first_shared": config(
        [par(l=left(heads=6, kv=3, dim=4, vdim=20, conv=2, size=5, rot=2, cap=3.0),
             r=right(heads=2, dim=6, vdim=6, decay=(0.3, 0.999))),
         gru(n=8), dict(par(l=left(heads=6, kv=3, dim=4, vdim=20, conv=2, size=5, rot=2,
                                   cap=3.0),
                            r=right(heads=2, dim=6, vdim=6, decay=(0.3, 0.999))),
                        weights_of=0)], width=24, vocab=33, taps=6, scale=1.0),
    "chunk_of_one": config([par(l=left(size=1)), wkv(heads=4, dim=4)], width=16),
    "big_chunk": config([par(l=left(size=1000)), gru()], width=16),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(tmp_path, device, name):
    cfg = OTHER[name]
    d, W = model_dir(tmp_path, cfg, seed=12)
    toks = tokens(53, cfg["vocab"], 7)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [19, 2, 6, 1]), want)


def test_lowrank_size_comes_from_the_checkpoint(tmp_path):
    cfg = config([wkv()])
    W = oracle.random_weights(cfg, 13)
    g = torch.Generator().manual_seed(0)
    W["l0.mix.w1"] = (torch.randn(5, 32, generator=g) * 0.2).bfloat16()
    W["l0.mix.w2"] = (torch.randn(24, 5, generator=g) * 0.4).bfloat16()
    d, W = model_dir(tmp_path, cfg, seed=13, W=W)
    toks = tokens(20, cfg["vocab"], 8)
    check(replay(engine(d, "cpu"), "a", toks, [20]), oracle.forward(cfg, W, toks))


def test_unconsumed_tensor_is_an_error(tmp_path):
    cfg = config([gru()])
    W = oracle.random_weights(cfg, 14)
    W["l0.mix.extra"] = torch.zeros(3).bfloat16()
    d, _ = model_dir(tmp_path, cfg, seed=14, W=W)
    with pytest.raises(ValueError):
        engine(d, "cpu")


# ---------------------------------------------------------------------------
# generation through the engine's own entry point and scheduler
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=15)
    eng = LLMEngine(EngineConfig(
        model=d, device=device, dtype="float32", num_gpu_blocks=32, max_num_seqs=3,
        max_model_len=256, max_num_batched_tokens=24))  # prompts get chunked
    prompts = {"p%d" % i: tokens(n, MIXED["vocab"], 50 + i)
               for i, n in enumerate([31, 5, 47, 12, 2])}
    for rid, t in prompts.items():
        eng.add_request(t, SamplingParams(max_tokens=12, ignore_eos=True), request_id=rid)
    done = {}
    for _ in range(400):
        if not eng.has_work():
            break
        for o in eng.step():
            if o.finished:
                done[o.request_id] = list(o.output_token_ids)
    assert set(done) == set(prompts)
    for rid, t in prompts.items():
        gen = done[rid]
        assert len(gen) == 12
        logits = oracle.forward(MIXED, W, t + gen)
        for i, tok in enumerate(gen):
            row = logits[len(t) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (rid, i)
    assert eng.state_manager.num_free == 3
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graph_replays_match_oracle(tmp_path, dtype):
    """Pure-decode steps replay a captured graph; prompt portions of later
    arrivals run eagerly between replays. Every generated token is checked."""
    d, W = model_dir(tmp_path, MIXED, seed=17)
    eng = LLMEngine(EngineConfig(
        model=d, device="cuda", dtype=dtype, num_gpu_blocks=64, max_num_seqs=6,
        max_model_len=512, max_num_batched_tokens=64, enable_graphs=True))
    prompts = {"g%d" % i: tokens(n, MIXED["vocab"], 90 + i)
               for i, n in enumerate([9, 33, 4, 70, 18, 2, 25])}
    pending = list(prompts.items())
    done, steps = {}, 0
    while (pending or eng.has_work()) and steps < 500:
        if pending and steps % 5 == 0:  # arrivals interleave with decode steps
            rid, t = pending.pop(0)
            eng.add_request(t, SamplingParams(max_tokens=24, ignore_eos=True),
                            request_id=rid)
        for o in eng.step():
            if o.finished:
                done[o.request_id] = list(o.output_token_ids)
        steps += 1
    assert eng.runner._graphs, "no decode graph was captured"
    assert set(done) == set(prompts)
    tol = 1e-3 if dtype == "float32" else 0.25
    for rid, t in prompts.items():
        gen = done[rid]
        logits = oracle.forward(MIXED, W, t + gen)
        for i, tok in enumerate(gen):
            row = logits[len(t) - 1 + i]
            assert row[tok] >= row.max() - tol * row.std(), (rid, i)


def test_state_slots_survive_preemption_and_abort(tmp_path):
    d, W = model_dir(tmp_path, MIXED, seed=16)
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
    for rid in ("q0", "q2"):
        gen = done[rid]
        logits = oracle.forward(MIXED, W, prompts[rid] + gen)
        for i, tok in enumerate(gen):
            row = logits[len(prompts[rid]) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std()
    assert eng.state_manager.num_free == 3


def test_served_over_http_with_sampling():
    """The family behind the engine's OpenAI server: greedy and sampled
    completions through the same scheduler, sampler and tokenizer plumbing."""
    from fastapi.testclient import TestClient

    from kubeai_amd.engine.server import EngineServer, build_app

    cfg = EngineConfig(model="dulotar-tiny", device="cpu", num_gpu_blocks=64,
                       max_model_len=256, max_num_seqs=4)
    server = EngineServer(cfg, "hybrid")
    server.start()
    server._ready.wait(timeout=60)
    try:
        with TestClient(build_app(server)) as c:
            r = c.post("/v1/completions", json={"model": "hybrid", "prompt": "a b c d e",
                                                "max_tokens": 6, "temperature": 0})
            assert r.status_code == 200, r.text
            greedy = r.json()
            assert greedy["usage"]["completion_tokens"] >= 1
            r2 = c.post("/v1/completions", json={"model": "hybrid", "prompt": "a b c d e",
                                                 "max_tokens": 6, "temperature": 0})
            assert r2.json()["choices"][0]["text"] == greedy["choices"][0]["text"]
            r3 = c.post("/v1/completions", json={"model": "hybrid", "prompt": "a b c d e",
                                                 "max_tokens": 6, "temperature": 0.9,
                                                 "top_p": 0.9, "seed": 3})
            assert r3.status_code == 200, r3.text
    finally:
        server.stop()
