"""Bozevik in the engine against the plain implementation in tests/bozevik_oracle.py (no shared code).

Every test makes its own small configuration and random bf16 weights, writes them as a checkpoint directory
(config.json + model.safetensors), loads that through the engine's own loader, and drives the engine's step
function (LLMEngine.replay_step for dictated steps, LLMEngine.generate / step for scheduled ones).  Each test runs
on the CPU (torch reference ops) and, marked gpu, on the MI355X (HIP kernels), in bf16 and in fp32.

Error measure: per position, the rms over the vocabulary of the logit difference (mean removed), relative to the
rms of the oracle's logits.  fp32 must agree to rounding (1e-4); bf16 to a few roundings per layer (4e-2).
"""
import json
import math
import os

import pytest
import torch

import bozevik_oracle as O

from symmetry_amd import ops
from symmetry_amd.engine.llm_engine import EngineConfig, LLMEngine
from symmetry_amd.engine.sequence import SamplingParams

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {"float32": 1e-4, "bfloat16": 4e-2}
BS = 16  # cache block size of the test engines


def _device(name):
    if name == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return name


def _cfg_a():
    """Sizes all different from one another; owner / borrower / owner; dense, routed (top 2 of 5, shared), none."""
    return O.make_config(width=72, vocab=112, eps=1e-5, logit_scale=1.7, layers=[
        {"type": "latent_attention", "mixer": O.mixer(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=40, q_rank=28, base=5000.0, scale=0.21),
         "mlp": O.dense(ff=88, limit=1.25)},
        {"type": "latent_attention", "mixer": O.mixer(heads=2, dim=16, rot_dim=8, vdim=12, kv_rank=40, q_rank=20, base=5000.0, scale=0.3, kv_from=0),
         "mlp": O.moe(experts=5, top=2, ff=24, limit=1.0, shared_ff=40, shared_limit=2.5)},
        {"type": "latent_attention", "mixer": O.mixer(heads=4, dim=8, rot_dim=8, vdim=8, kv_rank=40, q_rank=36, base=5000.0, scale=0.25),
         "mlp": None},
        {"type": "latent_attention", "mixer": O.mixer(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=40, q_rank=28, base=5000.0, scale=0.2, kv_from=2),
         "mlp": O.moe(experts=3, top=3, ff=16, limit=0.75, shared_ff=0)},
    ])


def _cfg_b():
    """One layer of each feed-forward kind, odd sizes (nothing a multiple of 8 but the rotary), top 1; a third layer
    with a cache row of another width, rotary base and length than the first."""
    return O.make_config(width=50, vocab=77, eps=1e-6, logit_scale=1.0, layers=[
        {"type": "latent_attention", "mixer": O.mixer(heads=1, dim=10, rot_dim=6, vdim=14, kv_rank=70, q_rank=18, base=300.0, scale=0.4),
         "mlp": O.moe(experts=4, top=1, ff=22, limit=1.5, shared_ff=26, shared_limit=0.5)},
        {"type": "latent_attention", "mixer": O.mixer(heads=5, dim=6, rot_dim=6, vdim=6, kv_rank=70, q_rank=30, base=300.0, scale=0.35, kv_from=0),
         "mlp": O.dense(ff=33, limit=2.0)},
        {"type": "latent_attention", "mixer": O.mixer(heads=2, dim=4, rot_dim=10, vdim=9, kv_rank=22, q_rank=12, base=90.0, scale=0.5),
         "mlp": O.dense(ff=20, limit=1.0)},
    ])


def _cfg_c():
    """Latent 48 + rotary 16 (a 64-wide cache row: the shapes the MFMA attention kernel takes in bf16), 5 and 18 heads."""
    return O.make_config(width=64, vocab=128, eps=1e-5, logit_scale=0.8, layers=[
        {"type": "latent_attention", "mixer": O.mixer(heads=5, dim=8, rot_dim=16, vdim=12, kv_rank=48, q_rank=24, base=1000.0, scale=0.3),
         "mlp": O.dense(ff=64, limit=3.0)},
        {"type": "latent_attention", "mixer": O.mixer(heads=18, dim=8, rot_dim=16, vdim=4, kv_rank=48, q_rank=40, base=1000.0, scale=0.25, kv_from=0),
         "mlp": O.moe(experts=4, top=2, ff=32, limit=1.0, shared_ff=32, shared_limit=1.0)},
    ])


def _cfg_d():
    """Width 128 with 64-wide experts: bf16 on the GPU runs the expert products on the MFMA grouped GEMM."""
    return O.make_config(width=128, vocab=160, eps=1e-5, logit_scale=1.2, layers=[
        {"type": "latent_attention", "mixer": O.mixer(heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=48, q_rank=32, base=1000.0, scale=0.2),
         "mlp": O.moe(experts=6, top=2, ff=64, limit=1.5, shared_ff=128, shared_limit=2.0)},
    ])


def _checkpoint(tmp_path, cfg, seed=0, tensors=None):
    from safetensors.torch import save_file

    tensors = tensors or O.random_tensors(cfg, seed)
    d = os.path.join(str(tmp_path), f"ckpt{seed}")
    os.makedirs(d, exist_ok=True)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(d, "model.safetensors"))
    return d, tensors


def _engine(path, device, dtype, blocks=40, seqs=4, **kw):
    base = dict(model="bozevik-test", weights=path, device=device, dtype=dtype, max_num_seqs=seqs, block_size=BS,
                num_kv_blocks=blocks + 1, max_model_len=blocks * BS, enable_prefix_caching=False)
    base.update(kw)
    return LLMEngine(EngineConfig(**base))


def _err(got, want):
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.double().pow(2).mean().sqrt()).max())


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _clear_tokens(cfg, tensors, n, seed, margin=0.08):
    """Token ids whose routing is no close call anywhere (every router's last chosen logit leads the first rejected
    one by ``margin``): bf16 activations may resolve a near-tie the other way, which is no fault of the engine."""
    for s in range(seed, seed + 200):
        ids = _tokens(n, cfg["vocab"], s)
        O.ROUTER_MARGINS = []
        try:
            O.forward(cfg, tensors, ids, torch.float64)
            if all(m > margin for m in O.ROUTER_MARGINS):
                return ids
        finally:
            O.ROUTER_MARGINS = None
    raise AssertionError("no token sequence without a routing near-tie in 200 seeds")


def _replay(eng, plan, requests):
    """plan: list of steps, each a list of (request name, token count).  Every position's logits are asked for.
    Returns {name: logits [len, V]}."""
    at = {k: 0 for k in requests}
    got = {k: [] for k in requests}
    for step in plan:
        entries, end = [], []
        for name, n in step:
            lo = at[name]
            entries.append((name, requests[name][lo:lo + n], list(range(n))))
            at[name] = lo + n
            if at[name] == len(requests[name]):
                end.append(name)
        lg = eng.replay_step(entries, end)
        r = 0
        for name, n in step:
            got[name].append(lg[r:r + n])
            r += n
    return {k: torch.cat(v) for k, v in got.items() if v}


def _oracle(cfg, tensors, ids):
    return O.forward(cfg, tensors, ids, torch.float64)


# ---- whole prompts, decoding, portions ----------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("make", [_cfg_a, _cfg_b, _cfg_c, _cfg_d])
def test_prompt_decode_and_portions_agree_with_oracle(tmp_path, device, dtype, make):
    device = _device(device)
    cfg = make()
    path, tensors = _checkpoint(tmp_path, cfg)
    eng = _engine(path, device, dtype)
    ids = _clear_tokens(cfg, tensors, (3 if make is not _cfg_c else 9) * BS + 5, 1)   # (_cfg_c: past one 64-row query tile)
    want = _oracle(cfg, tensors, ids)
    n = len(ids)
    plans = {
        "whole": [[("a", n)]],
        "token by token": [[("a", 1)] for _ in range(n)],
        "prompt then decode": [[("a", BS + 3)]] + [[("a", 1)] for _ in range(n - BS - 3)],
        # portions of 2, of a block, across block edges, and a single token in between
        "portions": [[("a", k)] for k in (2, BS, 2, 1, BS - 1, 3, 2)] + [[("a", n - (2 * BS + 9))]],
    }
    for name, plan in plans.items():
        got = _replay(eng, plan, {"a": ids})["a"]
        assert got.shape == want.shape
        assert _err(got, want) < TOL[dtype], (name, _err(got, want))
    # every block and slot went back to the pools
    assert eng.blocks.num_free == eng.blocks.num_blocks - 1 and eng.slots.num_free == 4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_of_blocks_and_slots(tmp_path, device, dtype):
    """Unequal requests side by side (portions beside single tokens, a request that pauses), in a pool too small to
    hold them all at once without reuse: 4 slots, and blocks that earlier requests freed."""
    device = _device(device)
    cfg = _cfg_a()
    path, tensors = _checkpoint(tmp_path, cfg, seed=3)
    eng = _engine(path, device, dtype, blocks=12)
    reqs = {k: _clear_tokens(cfg, tensors, n, 100 * i) for i, (k, n) in
            enumerate([("a", 1), ("b", 37), ("c", 2 * BS), ("d", 9), ("e", 50), ("f", BS + 1), ("g", 3)])}
    plan = [
        [("b", 20), ("a", 1), ("c", 2), ("d", 1)],
        [("b", 1), ("c", BS - 2), ("d", 1), ("e", 7)],          # a ended: its slot goes to e
        [("c", 1), ("d", 5), ("e", 2)],                        # b pauses
        [("b", 16), ("c", BS - 1), ("d", 2), ("e", 30)],       # b, c, d end here
        [("e", 1), ("f", BS + 1), ("g", 2)],
        [("e", 10), ("g", 1)],
    ]
    got = _replay(eng, plan, reqs)
    for k, ids in reqs.items():
        want = _oracle(cfg, tensors, ids)
        assert _err(got[k], want) < TOL[dtype], (k, _err(got[k], want))
    assert eng.blocks.num_free == eng.blocks.num_blocks - 1 and eng.slots.num_free == 4
    # and the same requests alone give the same logits as in the batch (beyond rounding)
    alone = _replay(eng, [[("e", 50)]], {"e": reqs["e"]})["e"]
    assert _err(got["e"], alone) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_through_graph_buckets(tmp_path, device):
    """A short prompt, then 150 single-token steps across many block edges (on the GPU: replayed hipGraphs whose
    context bucket grows), with a second sequence joining and leaving the decode batch."""
    device = _device(device)
    cfg = _cfg_b()
    path, tensors = _checkpoint(tmp_path, cfg, seed=5)
    eng = _engine(path, device, "float32", blocks=24)
    a, b = _tokens(155, cfg["vocab"], 2), _tokens(40, cfg["vocab"], 3)
    plan = [[("a", 5)]] + [[("a", 1)] for _ in range(30)] + [[("a", 1), ("b", 9)]] + \
        [[("a", 1), ("b", 1)] for _ in range(31)] + [[("a", 1)] for _ in range(88)]
    got = _replay(eng, plan, {"a": a, "b": b})
    assert _err(got["a"], _oracle(cfg, tensors, a)) < TOL["float32"]
    assert _err(got["b"], _oracle(cfg, tensors, b)) < TOL["float32"]


# ---- faults that random weights hide --------------------------------------------------------------------
def _spiked(cfg, seed, layer=0):
    """Weights whose layer-`layer` attention is sharp: the shared rotary key part and the queries are scaled up, so one
    or two keys take nearly all of each softmax and a key that is dropped, shifted by one, or leaked from the future
    changes the logits by far more than the tolerance."""
    t = O.random_tensors(cfg, seed)
    p = f"l{layer}.mix."
    t[p + "uq"] = (t[p + "uq"].float() * 6).to(torch.bfloat16)
    t[p + "dkv.norm"] = (t[p + "dkv.norm"].float() * 3).to(torch.bfloat16)
    return t


@pytest.mark.parametrize("device", DEVICES)
def test_sharp_attention_far_keys_and_block_edges(tmp_path, device):
    device = _device(device)
    cfg = _cfg_a()
    path, tensors = _checkpoint(tmp_path, cfg, seed=7, tensors=_spiked(cfg, 7))
    eng = _engine(path, device, "float32", blocks=40)
    ids = _tokens(20 * BS + 3, cfg["vocab"], 4)
    want = _oracle(cfg, tensors, ids)
    # the oracle itself must be sensitive: dropping the first token changes late logits visibly
    assert _err(_oracle(cfg, tensors, ids[1:])[-8:], want[-8:]) > 50 * TOL["float32"]
    n = len(ids)
    for name, plan in {
        "whole": [[("a", n)]],
        "portions cut at and around block edges": [[("a", k)] for k in (BS - 1, 2, BS, BS + 1, 2 * BS - 2, 7 * BS)] +
                                                   [[("a", n - 12 * BS - 40)]] + [[("a", 1)] for _ in range(40)],
    }.items():
        got = _replay(eng, plan, {"a": ids})["a"]
        assert _err(got, want) < TOL["float32"], (name, _err(got, want))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attn_op_picks_exactly_the_visible_keys(device, dtype):
    """The attention op alone, on a crafted cache: for a query at position p, a key made to dominate the softmax must
    be returned when it sits at 0, at a block's last / first row, at p - 1 or at p, and must have no effect at p + 1;
    with scattered, non-monotonic block tables."""
    device = _device(device)
    g = torch.Generator().manual_seed(0)
    H, r, rot, nb = 3, 48, 16, 12     # a 64-wide row: bf16 on the GPU takes the MFMA kernel, fp32 the wave kernel
    Dk = r + rot
    cache = (torch.randn(nb, BS, Dk, generator=g) * 0.1)
    table = torch.tensor([[7, 2, 9, 4, 11, 1], [3, 10, 5, 8, 6, 0]], dtype=torch.int32)
    q = torch.randn(2, H, Dk, generator=g) * 0.1
    u = torch.zeros(Dk)
    u[5], u[r + 3] = 1.0, 1.0            # one latent direction and one rotary-part direction
    q = q + 40.0 * u
    for p, seq in ((5 * BS + 7, 0), (2 * BS, 1), (BS - 1, 0), (0, 1)):
        for j in sorted({0, BS - 1, BS, BS + 1, p - 1, p, p + 1, 4 * BS}):
            if j < 0 or j >= 6 * BS:
                continue
            c = cache.clone()
            c[table[seq, j // BS], j % BS] += 3.0 * u
            out = torch.zeros(2, H, r, dtype=dtype)
            pos = torch.tensor([p, 0], dtype=torch.int32) if seq == 0 else torch.tensor([0, p], dtype=torch.int32)
            row_seq = torch.tensor([0, 1], dtype=torch.int32)
            args = [t.to(device) for t in (q.to(dtype), c.to(dtype), table, row_seq, pos)]
            o = out.to(device)
            ops.latent_attn(*args, 1.0, r, o)
            got = o[seq].float().cpu()
            # plain softmax over the visible keys
            rows = c.to(dtype).float()[table[seq].long()].reshape(-1, Dk)[: p + 1]
            w = torch.softmax(q[seq].to(dtype).float() @ rows.t(), -1)
            want = w @ rows[:, :r]
            assert torch.allclose(got, want, atol=2e-2 if dtype == torch.bfloat16 else 1e-5), (p, j)
            if j <= p:
                assert float(w[:, j].min()) > 0.99           # the crafted key took the softmax ...
            else:
                base = torch.softmax(q[seq].to(dtype).float() @ cache.to(dtype).float()[table[seq].long()].reshape(-1, Dk)[: p + 1].t(), -1)
                assert torch.allclose(w, base)                # ... and one past the query changes nothing


@pytest.mark.gpu
@pytest.mark.parametrize("H,r,rot", [(1, 16, 16), (5, 48, 16), (20, 96, 32), (70, 64, 64), (3, 512, 64), (40, 512, 64)])
def test_latent_attn_mfma_forms_against_the_wave_kernel(H, r, rot):
    """Prompt tiles (several runs that start mid-sequence, partial 64-row tiles, scattered blocks) and the decode form
    with split-KV partitions, MFMA kernel vs the one-wave kernel and vs a plain softmax."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev, g = "cuda", torch.Generator().manual_seed(H)
    Dk, bs, nb = r + rot, 16, 80
    cache = torch.randn(nb, bs, Dk, generator=g).to(torch.bfloat16)
    runs = [(300, 130), (0, 70), (517, 1), (64, 64)]                      # (first position, rows) per sequence
    perm = torch.randperm(nb - 1, generator=g) + 1
    mb = 40
    table = torch.zeros(len(runs), mb, dtype=torch.int32)
    used = 0
    for i, (p0, n) in enumerate(runs):
        need = -(-(p0 + n) // bs)
        table[i, :need] = perm[used % 8:used % 8 + need].int()          # overlapping block sets are fine for a read-only op
        used += 3
    pos = torch.cat([torch.arange(p0, p0 + n) for p0, n in runs]).int()
    row_seq = torch.cat([torch.full((n,), i) for i, (_, n) in enumerate(runs)]).int()
    cu = torch.tensor([0] + list(torch.tensor([n for _, n in runs]).cumsum(0)), dtype=torch.int32)
    tiles = torch.tensor([(i, o) for i, (_, n) in enumerate(runs) for o in range(0, n, 64)] + [(0, 1 << 24)], dtype=torch.int32)
    T = int(pos.numel())
    q = (torch.randn(T, H, Dk, generator=g) * 0.5).to(torch.bfloat16)
    scale = 0.2
    want = torch.zeros(T, H, r)
    flat = cache.float()
    for t in range(T):
        rows = flat[table[row_seq[t]].long()].reshape(-1, Dk)[: int(pos[t]) + 1]
        want[t] = torch.softmax(q[t].float() @ rows.t() * scale, -1) @ rows[:, :r]
    d = lambda t: t.to(dev)
    outs = {}
    for name, kw in {"wave": dict(impl=1), "tiles": dict(tiles=d(tiles), cu_q=d(cu), impl=0), "rows": dict(impl=0)}.items():
        o = torch.zeros(T, H, r, dtype=torch.bfloat16, device=dev)
        used_impl = ops.latent_attn(d(q), d(cache), d(table), d(row_seq), d(pos), scale, r, o, **kw)
        assert used_impl == (1 if name == "wave" else 0)
        outs[name] = o.float().cpu()
        assert float((outs[name] - want).abs().max()) < 3e-2, name
    # split-KV partitions (decode form): rows of different sequences, context far past one partition
    sel = torch.tensor([129, 130 + 69, 200, 201 + 63])                    # last rows of the four runs
    for impl, parts in ((0, 3), (1, 3), (0, 10), (1, 10), (0, 20)):
        o = torch.zeros(4, H, r, dtype=torch.bfloat16, device=dev)
        po = torch.zeros(4, H, parts, r, device=dev)
        pml = torch.zeros(4, H, parts, 2, device=dev)
        ops.latent_attn(d(q[sel]), d(cache), d(table), d(torch.arange(4).int()), d(pos[sel]), scale, r, o, po, pml, impl=impl)
        assert float((o.float().cpu() - want[sel]).abs().max()) < 3e-2, (impl, parts)


# ---- each mechanism alone: op vs oracle function ------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_and_carried_state(device):
    device = _device(device)
    g = torch.Generator().manual_seed(1)
    d, T = 40, 9
    x = torch.randn(T, d, generator=g)
    mu = torch.rand(d, generator=g)
    want = O.token_shift(x, mu)
    # rows 0..3 in one step (first token of the sequence), rows 4..8 in the next, with the state in slot 2
    state = torch.full((3, d), 7.0)
    h = torch.zeros(T, d)
    dev = lambda t: t.to(device)
    s, hd = dev(state), dev(h)
    ops.token_shift(dev(x[:4]), dev(mu), dev(torch.tensor([-1, 0, 1, 2], dtype=torch.int32)), s, hd[:4])
    w1 = torch.ones(d)
    delta = torch.randn(4, d, generator=g)
    xs = dev(x[:4].clone())
    ops.add_layer_norm(dev(delta), dev(w1), 1e-5, xs, dev(torch.tensor([-1, -1, -1, 2], dtype=torch.int32)), s)
    assert torch.equal(s[2].cpu(), x[3]) and float(s[0].cpu()[0]) == 7.0      # the OLD row 3 was saved, slot 0 untouched
    assert torch.allclose(xs.cpu(), x[:4] + O.layer_norm(delta, w1, 1e-5), atol=1e-5)
    ops.token_shift(dev(x[4:]), dev(mu), dev(torch.tensor([-(2 + 2), 0, 1, 2, 3], dtype=torch.int32)), s, hd[4:])
    assert torch.allclose(hd.cpu(), want, atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
def test_layer_norm_history_mix(device):
    device = _device(device)
    g = torch.Generator().manual_seed(2)
    T, d = 5, 33
    hist = torch.randn(4, T, d, generator=g)
    coef = torch.tensor([0.3, -0.2, 0.9])
    x, delta, w = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g) * 3 + 1, torch.randn(d, generator=g)
    xn = x + O.layer_norm(delta, w, 1e-6)
    want = coef[0] * hist[0] + coef[1] * hist[1] + coef[2] * xn
    hd, xd = hist.clone().to(device), x.clone().to(device)
    act = torch.zeros(T, d, device=device)
    ops.add_layer_norm(delta.to(device), w.to(device), 1e-6, xd, None, None, hd, coef.to(device), 2, act)
    assert torch.allclose(xd.cpu(), want, atol=1e-5) and torch.allclose(hd[2].cpu(), xn, atol=1e-5)
    assert torch.equal(hd[3].cpu(), hist[3]) and torch.allclose(act.cpu(), want, atol=1e-5)
    out = torch.zeros(2, d, device=device)
    ops.layer_norm(xd, torch.tensor([4, 1], device=device), w.to(device), 1e-6, out)
    assert torch.allclose(out.cpu(), O.layer_norm(want[[4, 1]], w, 1e-6), atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_rotary_pairs_and_latent_prep(device):
    device = _device(device)
    g = torch.Generator().manual_seed(3)
    T, H, rot, rq, r, base = 6, 2, 8, 12, 20, 777.0
    pos = torch.tensor([0, 1, 5, 63, 64, 900], dtype=torch.int32)
    table = ops.rope_pair_table(1024, rot, base)
    src = torch.randn(T, H, 5 + rot, generator=g)
    dst = torch.zeros(T, H, 3 + rot)
    d_dev = dst.to(device)
    ops.rope_pairs(src.to(device)[:, :, 5:], d_dev[:, :, 3:], pos.to(device), table.to(device))
    want = O.rotate_pairs(src[:, :, 5:].double(), pos, base, rot)
    assert torch.allclose(d_dev.cpu()[:, :, 3:].double(), want, atol=2e-5) and float(d_dev[:, :, :3].abs().max()) == 0
    # latent_prep: both RMS norms, the rotary of the shared key part, rows written at their slots only
    z = torch.randn(T, rq + r + rot, generator=g)
    gq, gkv = torch.rand(rq, generator=g) + 0.5, torch.rand(r, generator=g) + 0.5
    slots = torch.tensor([3, 17, -1, 0, 31, 8], dtype=torch.int32)
    cache = torch.zeros(2, BS, r + rot)
    cq = torch.zeros(T, rq)
    cd, qd = cache.to(device), cq.to(device)
    ops.latent_prep(z.to(device), rq, r, rot, gq.to(device), gkv.to(device), 1e-5, pos.to(device), slots.to(device),
                    table.to(device), qd, cd)
    assert torch.allclose(qd.cpu(), O.rms_unit(z[:, :rq], 1e-5) * gq, atol=1e-5)
    rows = cd.cpu().view(-1, r + rot)
    c = O.rms_unit(z[:, rq:rq + r], 1e-5) * gkv
    kr = O.rotate_pairs(z[:, rq + r:].double(), pos, base, rot).float()
    for t in range(T):
        if slots[t] >= 0:
            assert torch.allclose(rows[slots[t]], torch.cat([c[t], kr[t]]), atol=2e-5)
    written = set(int(s) for s in slots if s >= 0)
    assert all(float(rows[i].abs().max()) == 0 for i in range(2 * BS) if i not in written)


@pytest.mark.parametrize("device", DEVICES)
def test_clamped_glu_and_routed_experts(device):
    device = _device(device)
    g = torch.Generator().manual_seed(4)
    T, d, E, k, F = 37, 24, 6, 3, 10
    x = torch.randn(T, d, generator=g)
    p = {"router": torch.randn(E, d, generator=g)}
    for e in range(E):
        p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"] = (torch.randn(F, d, generator=g), torch.randn(F, d, generator=g),
                                                           torch.randn(d, F, generator=g))
    mlp = {"router": {"experts": E, "top": k}, "expert": {"ff": F, "limit": 0.8}}
    want = O.moe_ff(p, "", mlp, x)
    # the weight scales the expert's INPUT: with clamps that differs from scaling its output
    s = torch.sigmoid(x @ p["router"].T).topk(k, -1)
    other = sum(s.values[:, j:j + 1] * torch.stack([O.glu_ff(p, f"e{int(s.indices[t, j])}.", x[t:t + 1], 0.8)[0] for t in range(T)])
                for j in range(k))
    assert _err(other, want) > 1e-2
    dev = lambda t: t.to(device)
    i32 = torch.int32
    R = T * k
    ids, w = torch.zeros(R, dtype=i32, device=device), torch.zeros(R, device=device)
    offsets, cursor = torch.zeros(E + 1, dtype=i32, device=device), torch.ones(E, dtype=i32, device=device)
    dst, xs = torch.zeros(R, dtype=i32, device=device), torch.zeros(R, d, device=device)
    ops.sigmoid_topk(dev(x), dev(p["router"]), k, ids, w)
    assert torch.equal(ids.cpu().view(T, k).sort(-1).values, s.indices.int().sort(-1).values)
    ops.expert_offsets(ids, R, E, offsets, cursor)
    ops.scatter_scaled(dev(x), ids, w, k, offsets, cursor, xs, dst)
    assert sorted(dst.cpu().tolist()) == list(range(R))
    w13 = torch.stack([torch.cat([p[f"e{e}.gate"], p[f"e{e}.up"]], 0) for e in range(E)])
    w2 = torch.stack([p[f"e{e}.down"] for e in range(E)])
    y1, act, y2 = torch.zeros(R, 2 * F, device=device), torch.zeros(R, F, device=device), torch.zeros(R, d, device=device)
    ops.grouped_linear(xs, dev(w13), offsets, y1)
    ops.clamped_glu(y1, 0.8, 1.702, act)
    ops.grouped_linear(act, dev(w2), offsets, y2)
    out = torch.zeros(T, d, device=device)
    ops.gather_sum(y2, dst, k, None, out)
    assert _err(out.cpu(), want) < 1e-5


# ---- the engine's own entry point and scheduler ---------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(tmp_path, device, dtype):
    """add_request / step: the scheduler forms the batches (prefill, mixed, pipelined decode), the engine samples
    greedily; every token must be the oracle's best next token for the text so far (up to near-ties)."""
    device = _device(device)
    cfg = _cfg_a()
    path, tensors = _checkpoint(tmp_path, cfg, seed=11)
    eng = _engine(path, device, dtype, blocks=30, seqs=3, max_num_batched_tokens=64, mixed_prefill_tokens=24)
    prompts = [_tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate((5, 70, 33, 1, 18))]   # 5 requests, 3 slots
    seqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=12, ignore_eos=True)) for i, p in enumerate(prompts)]
    while eng.has_unfinished():
        eng.step()
    tol = 1e-3 if dtype == "float32" else 0.15
    for p, s in zip(prompts, seqs):
        assert len(s.output_ids) == 12
        lg = _oracle(cfg, tensors, p + s.output_ids[:-1])
        for j, t in enumerate(s.output_ids):
            row = lg[len(p) - 1 + j]
            assert float(row.max() - row[t]) <= tol * float(row.std()), (j, t, int(row.argmax()))
    assert eng.blocks.num_free == eng.blocks.num_blocks - 1 and eng.slots.num_free == 3


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_and_abort_return_blocks_and_slots(tmp_path, device):
    """A pool too small for every sequence's decoded tail: the scheduler preempts (blocks and state slot go back, the
    sequence is recomputed from its first token later, its carried state rebuilt by that prefill) and the outputs
    still follow the oracle; an aborted request frees its slot for a waiting one."""
    device = _device(device)
    cfg = _cfg_a()
    path, tensors = _checkpoint(tmp_path, cfg, seed=13)
    eng = _engine(path, device, "float32", blocks=8, seqs=3, max_num_batched_tokens=64)
    prompts = [_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate((30, 25, 33, 12))]
    seqs = [eng.add_request(f"p{i}", p, SamplingParams(max_tokens=28, ignore_eos=True)) for i, p in enumerate(prompts)]
    steps = 0
    while eng.has_unfinished() and steps < 3000:
        eng.step()
        steps += 1
        if steps == 6:
            eng.abort("p1")
    assert sum(s.num_preemptions for s in seqs) > 0
    for i, (p, s) in enumerate(zip(prompts, seqs)):
        if i == 1:
            continue
        assert len(s.output_ids) == 28
        lg = _oracle(cfg, tensors, p + s.output_ids[:-1])
        for j, t in enumerate(s.output_ids):
            row = lg[len(p) - 1 + j]
            assert float(row.max() - row[t]) <= 1e-3 * float(row.std()), (i, j, t, int(row.argmax()))
    assert eng.blocks.num_free == eng.blocks.num_blocks - 1 and eng.slots.num_free == 3


def test_registered_config_and_checkpoint_roundtrip(tmp_path):
    from symmetry_amd.models.config import bozevik_from_config, bozevik_to_config, resolve
    from symmetry_amd.models.weights import random_weights, save_bozevik_checkpoint

    c = resolve("tiny-bozevik")
    assert bozevik_from_config(bozevik_to_config(c), c.name).layers == c.layers
    w = random_weights(c, seed=1)
    save_bozevik_checkpoint(w, str(tmp_path / "ck"))
    eng = _engine(str(tmp_path / "ck"), "cpu", "float32")
    ids = _tokens(21, c.vocab_size, 0)
    cfgd = json.load(open(tmp_path / "ck" / "config.json"))
    got = _replay(eng, [[("a", 13)], [("a", 8)]], {"a": ids})["a"]
    assert _err(got, _oracle(cfgd, w.tensors, ids)) < TOL["float32"]
    with pytest.raises(ValueError):
        bad = bozevik_to_config(c)
        bad["layers"][0]["mixer"]["window"] = 4
        bozevik_from_config(bad)
