"""Lemunex through the engine and op by op, against the plain oracle in tests/lemunex_oracle.py.

Every test builds its own small configuration and random weights (sizes all different from one another and from any
shipped checkpoint), writes them as a checkpoint, loads that through the engine, and compares with the oracle.  The CPU
runs use the torch reference ops, the ``gpu`` ones the HIP kernels; float32 comparisons are tight (rounding only),
bfloat16 ones use the spread that bf16 rounding gives.  A dictated step goes through LLMEngine.replay_step, i.e. the
scheduler, the block / slot managers, the runner's packed metadata (and decode hipGraphs on the GPU) and model.forward.
"""
from __future__ import annotations

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import lemunex_oracle as O  # noqa: E402

from symmetry_amd import ops  # noqa: E402
from symmetry_amd.engine.llm_engine import EngineConfig, LLMEngine  # noqa: E402
from symmetry_amd.engine.sequence import SamplingParams  # noqa: E402
from symmetry_amd.models import config as C  # noqa: E402
from symmetry_amd.models.weights import lemunex_random_weights, save_lemunex_checkpoint  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def say(*a):
    print(*a, flush=True)


# ---- configurations ---------------------------------------------------------------------------------------------
def attn(heads=4, kv=2, dim=24, vdim=8, window=5, rot=8, scaling=True, scale=0.3):
    r = C.RotarySpec(rot, 100.0, 3.0, 64.0, 8.0, 1.0) if scaling else C.RotarySpec(rot, 50.0)
    return C.WindowAttnSpec(heads, kv, dim, vdim, window, scale, r)


def pair(left=None, heads=3, dim=8, vdim=16, tau=4.0, rank=5, ls=0.7, rs=1.3):
    return C.PairMixerSpec(left or attn(), C.GatedLinearAttnSpec(heads, dim, vdim, tau, rank), ls, rs)


def ssm(heads=4, vdim=8, state=6, groups=2, conv=3, norm_groups=2):
    return C.StateSpaceSpec(heads, vdim, state, groups, conv, norm_groups)


def cfg_mixed(width=48, vocab=61):
    """Every branch once: both layer types, dense / routed / no feed-forward, identity experts, shared expert or not."""
    layers = (
        C.LemunexLayer("parallel", pair(), C.ReluSqSpec(40)),
        C.LemunexLayer("mamba2", ssm(), C.RoutedSpec(5, 2, 2, 16, 24)),
        C.LemunexLayer("parallel", pair(attn(heads=2, kv=1, dim=10, vdim=12, window=9, rot=4, scaling=False),
                                        heads=2, dim=5, vdim=7, tau=9.0, rank=3), C.RoutedSpec(4, 0, 3, 8, 0)),
        C.LemunexLayer("mamba2", ssm(heads=3, vdim=5, state=9, groups=1, conv=5, norm_groups=1), None),
        C.LemunexLayer("mamba2", ssm(heads=2, vdim=16, state=4, groups=2, conv=2, norm_groups=4), C.RoutedSpec(3, 1, 1, 8, 8)),
    )
    return C.LemunexConfig(name="t-mixed", vocab_size=vocab, hidden_size=width, layers=layers, norm_eps=1e-5)


def cfg_tiled(width=64, vocab=97):
    """Head sizes that the tiled kernels take (multiples of 16 / 32), one kv head group of 4, window across blocks."""
    layers = (
        C.LemunexLayer("parallel", pair(attn(heads=8, kv=2, dim=32, vdim=32, window=40, rot=16), heads=2, dim=32, vdim=64,
                                        rank=4), C.RoutedSpec(4, 1, 2, 64, 0)),
        C.LemunexLayer("mamba2", ssm(heads=4, vdim=32, state=64, groups=1, conv=4, norm_groups=1), C.ReluSqSpec(128)),
    )
    return C.LemunexConfig(name="t-tiled", vocab_size=vocab, hidden_size=width, layers=layers, norm_eps=1e-6)


def checkpoint(cfg, tmp_path, seed=0, sharpen=None):
    w = lemunex_random_weights(cfg, seed=seed)
    if sharpen:
        sharpen(w.tensors)
    path = str(tmp_path / f"{cfg.name}-{seed}")
    save_lemunex_checkpoint(w, path)
    return path, C.lemunex_to_config(cfg), {k: v.to(torch.bfloat16) for k, v in w.tensors.items()}


def engine(path, device, dtype, blocks=24, seqs=4, block_size=16, graphs=True):
    return LLMEngine(EngineConfig(model="t", weights=path, dtype=dtype, device=device, max_num_seqs=seqs,
                                  block_size=block_size, num_kv_blocks=blocks + 1, max_model_len=blocks * block_size,
                                  max_num_batched_tokens=8192, use_graphs=graphs, enable_prefix_caching=False,
                                  pipeline=False))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def run_schedule(eng, prompts: dict, schedule: list) -> dict:
    """schedule: steps of [(request, tokens this step)]; every position's logits are asked for.  -> id -> [n, V]."""
    at = {r: 0 for r in prompts}
    got = {r: [] for r in prompts}
    for step in schedule:
        entries, ends = [], []
        for r, n in step:
            lo = at[r]
            entries.append((r, prompts[r][lo:lo + n], list(range(n))))
            at[r] = lo + n
            if at[r] == len(prompts[r]):
                ends.append(r)
        lg = eng.replay_step(entries, ends)
        o = 0
        for r, n in step:
            got[r].append(lg[o:o + n].clone())
            o += n
    return {r: torch.cat(v) for r, v in got.items() if v}


def err(a, b):
    d = (a.double() - b.double())
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / b.double().std(-1).clamp_min(1e-6)).max())


TOL = {"float32": 2e-4, "bfloat16": 0.15}   # bf16: a lost mechanism gives errors near 1


def oracle_logits(cj, W, toks):
    return O.forward(cj, W, toks).float()


def safe_rows(cj, W, toks, dtype, thresh=0.03):
    """Rows to compare: all of them in float32; in bfloat16 the rows before the first token at which some router's
    last chosen and first rejected outputs are closer than ``thresh`` (bf16 rounding may flip that choice, and the
    recurrent layers carry the difference to every later token)."""
    if dtype == "float32":
        return len(toks)
    margins = []
    O.forward(cj, W, toks, margins=margins)
    if not margins:
        return len(toks)
    close = (torch.stack(margins).min(0).values < thresh).nonzero()
    return int(close[0]) if len(close) else len(toks)


# ---- the whole model through the engine ------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("make", [cfg_mixed, cfg_tiled])
def test_prompt_decode_portions(tmp_path, device, dtype, make):
    """Whole prompt, prompt then token-by-token decoding, and portions down to two tokens all give the oracle's logits."""
    say("prompt/decode/portions", make.__name__, device, dtype)
    cfg = make()
    path, cj, W = checkpoint(cfg, tmp_path, sharpen=_decisive)
    toks = tokens(75, cfg.vocab_size, 1)
    want = oracle_logits(cj, W, toks)
    safe = safe_rows(cj, W, toks, dtype)
    assert safe >= 10, safe
    eng = engine(path, device, dtype)
    for name, cuts in (("whole", [75]), ("decode", [30] + [1] * 45), ("portions", [2, 3, 17, 2, 16, 1, 1, 5, 2, 26]),
                       ("tokens", [1] * 20)):
        say("  ", name)
        n = sum(cuts)
        got = run_schedule(eng, {"a": toks[:n]}, [[("a", c)] for c in cuts])["a"]
        m = min(n, safe)
        assert err(got[:m], want[:m]) < TOL[dtype], (name, err(got[:m], want[:m]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_pages_and_slots(tmp_path, device, dtype):
    """Unequal requests side by side (portions beside single tokens, a request that pauses), in a pool of three slots
    and few blocks that are freed and used again: every request's logits equal the oracle's for it alone."""
    say("mixed batches", device, dtype)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=3, sharpen=_decisive)
    P = {r: tokens(n, cfg.vocab_size, 10 + i) for i, (r, n) in enumerate([("a", 40), ("b", 23), ("c", 9), ("d", 31), ("e", 1),
                                                                           ("f", 18)])}
    sched = [[("a", 7), ("b", 2)], [("a", 1), ("b", 16), ("c", 3)], [("a", 16), ("c", 1)], [("b", 1), ("c", 1), ("a", 1)],
             [("a", 15), ("b", 4), ("c", 4)],                      # a, b, c end; their pages and slots go back
             [("d", 5), ("e", 1), ("f", 2)], [("d", 1), ("f", 1)], [("f", 15), ("d", 24)], [("d", 1)]]
    eng = engine(path, device, dtype, blocks=7, seqs=3)
    got = run_schedule(eng, P, sched)
    assert len(eng.blocks.free) == 7 and eng.slots.num_free == 3
    if dtype == "float32":
        for r, toks in P.items():
            e = err(got[r], oracle_logits(cj, W, toks))
            assert e < TOL[dtype], (r, e)
        return
    # bfloat16: against each request alone (whole prompt, its own engine), the same arithmetic without the batch
    alone = engine(path, device, dtype)
    for r, toks in P.items():
        ref = run_schedule(alone, {r: toks}, [[(r, len(toks))]])[r]
        m = safe_rows(cj, W, toks, dtype)
        if m:
            assert err(got[r][:m], ref[:m]) < 0.05, (r, err(got[r][:m], ref[:m]))
            assert err(ref[:m], oracle_logits(cj, W, toks)[:m]) < 3 * TOL[dtype]


def _decisive(t):
    """Peaked router scores: bf16 rounding does not flip a choice that carries weight."""
    for k in t:
        if k.endswith("mlp.router"):
            t[k] = t[k] * 8.0


def _sharp(t):
    """Attention that looks hard at single keys and recurrences that forget slowly: a key one place outside the window,
    or a state lost at a cut, moves the logits by far more than the tolerance."""
    for k in t:
        if k.endswith("left.q") or k.endswith("left.k"):
            t[k] = t[k] * 3.0
        if k.endswith("a2.b"):
            t[k] = t[k] + 2.0
        if k.endswith("dt_bias"):
            t[k] = t[k] - 1.0


@pytest.mark.parametrize("device", DEVICES)
def test_window_and_block_edges(tmp_path, device):
    """Sharp attention, cuts and decoding at and around the window's and the blocks' edges (float32)."""
    say("edges", device)
    cfg = cfg_tiled()
    path, cj, W = checkpoint(cfg, tmp_path, seed=5, sharpen=_sharp)
    toks = tokens(70, cfg.vocab_size, 7)
    want = oracle_logits(cj, W, toks)
    # dropping the oldest key of the window or adding the one before it must show: the oracle with window -+ 1 differs
    for dw in (-1, 1):
        cj2 = {**cj, "layers": [dict(L) for L in cj["layers"]]}
        import copy

        cj2 = copy.deepcopy(cj)
        cj2["layers"][0]["mixer"]["left"]["mask"]["size"] += dw
        assert err(oracle_logits(cj2, W, toks)[45:], want[45:]) > 50 * TOL["float32"]
    eng = engine(path, device, "float32", block_size=16)
    for cuts in ([39, 1, 1, 1, 28], [40, 30], [41, 29], [15, 1, 16, 1, 7] + [1] * 30, [16, 16, 8, 30]):
        assert sum(cuts) == len(toks)
        got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
        assert err(got, want) < TOL["float32"], (cuts, err(got, want))


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_and_far_state(tmp_path, device):
    """200 tokens decoded one by one after a short prompt, two sequences of different lengths in the batch; the
    recurrences carry the first tokens all the way (the oracle with the first token changed differs at the end)."""
    say("long decode", device)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=8, sharpen=_sharp)
    a, b = tokens(230, cfg.vocab_size, 20), tokens(120, cfg.vocab_size, 21)
    want_a, want_b = oracle_logits(cj, W, a), oracle_logits(cj, W, b)
    other = oracle_logits(cj, W, [(a[0] + 1) % cfg.vocab_size] + a[1:])
    assert err(other[-5:], want_a[-5:]) > 20 * TOL["float32"]
    eng = engine(path, device, "float32", blocks=30)
    sched = [[("a", 30), ("b", 3)]] + [[("a", 1), ("b", 1)]] * 117 + [[("a", 1)]] * 83
    got = run_schedule(eng, {"a": a, "b": b}, sched)
    assert err(got["a"], want_a) < TOL["float32"] and err(got["b"], want_b) < TOL["float32"]
    if device != "cpu":
        assert eng.runner.graph_replays > 0      # decode steps ran as replayed hipGraphs


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """engine.generate / step(): five requests, three slots, greedy; each output token is the oracle's argmax (tokens
    whose top two logits are closer than the tolerance are skipped)."""
    say("generate", device)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=11)
    eng = engine(path, device, "float32", blocks=12, seqs=3)
    prompts = [tokens(n, cfg.vocab_size, 30 + i) for i, n in enumerate((5, 19, 2, 33, 11))]
    outs = {}
    for i, p in enumerate(prompts):
        eng.add_request(f"r{i}", p, SamplingParams(max_tokens=12, ignore_eos=True))
    while eng.has_unfinished():
        for o in eng.step():
            if o.finished:
                outs[o.request_id] = list(o.seq.output_ids)
    for i, p in enumerate(prompts):
        out = outs[f"r{i}"]
        assert len(out) == 12
        lg = oracle_logits(cj, W, p + out[:-1])[len(p) - 1:]
        for j, t in enumerate(out):
            top = lg[j].topk(2).values
            assert float(lg[j].max() - lg[j][t]) <= 1e-3 * float(lg[j].std()) or float(top[0] - top[1]) < 1e-3, (i, j)


def test_config_reader_rejects_unknown_keys_and_roundtrips(tmp_path):
    cfg = cfg_mixed()
    path, cj, _ = checkpoint(cfg, tmp_path)
    from symmetry_amd.models.weights import safetensors_shapes

    again = C.from_config_json(cj, "t-mixed", safetensors_shapes(path))
    assert again == cfg
    bad = {**cj, "layers": [dict(cj["layers"][0], mixer=dict(cj["layers"][0]["mixer"], sink=1))] + cj["layers"][1:]}
    with pytest.raises(ValueError):
        C.from_config_json(bad, "x", safetensors_shapes(path))


# ---- mechanisms alone: op against oracle function ---------------------------------------------------------------
def _dev(device, *ts):
    return [t.to(device) if torch.is_tensor(t) else t for t in ts]


@pytest.mark.parametrize("device", DEVICES)
def test_rotary_table_and_window_attention(device):
    """qkv_rope_cache + window_attn on a paged cache against the oracle's attention: partial rotary with and without
    frequency scaling, grouped heads, a window crossing blocks, prompt rows and single rows, odd sizes."""
    say("op window_attn", device)
    torch.manual_seed(0)
    for (H, G, dk, dv, win, rot, scaling, n) in [(4, 2, 24, 8, 5, 8, True, 37), (6, 1, 10, 12, 70, 10, False, 90),
                                                  (8, 2, 32, 32, 33, 16, True, 100), (2, 2, 7, 3, 1, 2, True, 9),
                                                  (2, 1, 16, 24, 300, 8, True, 330), (2, 2, 8, 70, 600, 4, False, 640)]:
        spec = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "mask": {"size": win}, "scale": 0.41,
                "rot": {"base": 77.0, "dims": rot}}
        if scaling:
            spec["rot"]["scaling"] = {"factor": 5.0, "original": 50, "fast": 6.0, "slow": 0.5}
        d = 20
        W = {"q": torch.randn(H * dk, d) * 0.3, "k": torch.randn(G * dk, d) * 0.5, "v": torch.randn(G * dv, d), "g": torch.randn(H, d),
             "q.b": torch.randn(H * dk), "k.b": torch.randn(G * dk), "v.b": torch.randn(G * dv),
             "o": torch.eye(H * dv), "o.b": torch.zeros(H * dv)}
        W = {k: v.double() for k, v in W.items()}
        h = torch.randn(n, d).double()
        want = O.window_attention(W, "", spec, h).float()
        r = spec["rot"].get("scaling", {})
        table = ops.rope_scaled_table(n, rot, 77.0, r.get("factor", 0.0), r.get("original", 0.0), r.get("fast", 0.0),
                                      r.get("slow", 0.0))
        z = torch.cat([h @ W["q"].T, h @ W["k"].T, h @ W["v"].T, h @ W["g"].T], 1).float()
        bias = torch.cat([W["q.b"], W["k.b"], W["v.b"]]).float()
        BS = 8
        NB = n // BS + 3
        bt = (torch.randperm(NB - 1, generator=torch.Generator().manual_seed(n))[None] + 1).int()   # block 0 stays unused
        pos = torch.arange(n, dtype=torch.int32)
        slots = (bt[0][(pos // BS).long()] * BS + pos % BS).int()
        kc, vc = torch.zeros(NB, BS, G, dk), torch.zeros(NB, BS, G, dv)
        q, out = torch.empty(n, H, dk), torch.empty(n, H, dv)
        z, bias, table, bt, pos, slots, kc, vc, q, out = _dev(device, z, bias, table, bt, pos, slots, kc, vc, q, out)
        nq = H * dk + G * dk + G * dv
        ops.qkv_rope_cache(z[:, :nq], bias, H, G, dk, dv, pos, slots, table, q, kc, vc)
        row_seq = torch.zeros(n, dtype=torch.int32, device=device)
        ops.window_attn(q, kc, vc, bt, row_seq, pos, win, 0.41, z[:, nq:], out)
        assert torch.allclose(out.cpu().reshape(n, -1), want, atol=2e-4, rtol=2e-4), (H, G, dk, dv, win)


@pytest.mark.gpu
def test_window_attention_tiled_against_wave():
    """The tiled (MFMA) prompt kernel against the one-wave kernel on the same paged cache: several runs of unequal length
    that continue earlier context, windows shorter and longer than a key tile, heads sharing key / value heads."""
    say("op window tiled")
    torch.manual_seed(3)
    dev = "cuda"
    for (H, G, D, win, BS) in [(4, 2, 32, 40, 16), (8, 2, 96, 72, 64), (2, 1, 128, 1000, 64), (6, 6, 64, 5, 16)]:
        runs = [(0, 130), (37, 64), (200, 1), (64, 65), (5, 200)]          # (tokens already cached, new rows)
        NBs = [-(-(c + n) // BS) for c, n in runs]
        NB = sum(NBs) + 1
        perm = (torch.randperm(NB - 1) + 1).int()
        bt = torch.zeros(len(runs), max(NBs), dtype=torch.int32)
        o = 0
        for i, nb in enumerate(NBs):
            bt[i, :nb] = perm[o:o + nb]
            o += nb
        kc = torch.randn(NB, BS, G, D).bfloat16()
        vc = torch.randn(NB, BS, G, D).bfloat16()
        pos, row_seq, cu, tiles = [], [], [0], []
        for i, (c, n) in enumerate(runs):
            pos += list(range(c, c + n))
            row_seq += [i] * n
            cu.append(cu[-1] + n)
            tiles += [(i, r) for r in range(0, n, 64)]
        T_ = len(pos)
        q = (torch.randn(T_, H, D) * 0.5).bfloat16()
        gate = torch.randn(T_, H + 2).bfloat16()
        ti = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        args = [q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), ti(row_seq), ti(pos)]
        out = [torch.empty(T_, H, D, dtype=torch.bfloat16, device=dev) for _ in range(2)]
        g = gate.to(dev)[:, 1:H + 1]
        used = [ops.window_attn(*args, win, D ** -0.5, g, out[0], ti(tiles), ti(cu), impl=1),
                ops.window_attn(*args, win, D ** -0.5, g, out[1], None, None, impl=0)]
        assert used == [1, 0]
        assert torch.allclose(out[0].float(), out[1].float(), atol=0.02, rtol=0.02), (H, G, D, win)


@pytest.mark.parametrize("device", DEVICES)
def test_window_attention_edge_keys(device):
    """One key with a score far above all others, placed just inside / just outside the window and at block borders:
    the output is that key's value row exactly when it is visible."""
    say("op window edges", device)
    H, G, dk, dv, BS, NB, win = 2, 1, 16, 16, 8, 8, 12
    for p in (11, 12, 23, 24, 40):
        for back in (0, 1, 7, 8, win - 1, win):
            j = p - back
            if j < 0:
                continue
            kc, vc = torch.zeros(NB, BS, G, dk), torch.randn(NB, BS, G, dv)
            bt = torch.tensor([[5, 2, 7, 1, 3, 6, 0, 0]], dtype=torch.int32)
            slot = int(bt[0][j // BS]) * BS + j % BS
            kc.view(-1, G, dk)[slot, 0, 0] = 50.0
            q = torch.zeros(1, H, dk)
            q[:, :, 0] = 1.0
            out = torch.empty(1, H, dv)
            pos = torch.tensor([p], dtype=torch.int32)
            a = _dev(device, q, kc, vc, bt, torch.zeros(1, dtype=torch.int32), pos, out)
            ops.window_attn(a[0], a[1], a[2], a[3], a[4], a[5], win, 1.0, None, a[6])
            hit = torch.allclose(a[6].cpu()[0, 0], vc.view(-1, G, dv)[slot, 0], atol=1e-4)
            assert hit == (back < win), (p, back)


@pytest.mark.parametrize("device", DEVICES)
def test_decay_scan_both_modes_and_cuts(device):
    """decay_scan against the oracle's two recurrences, in one run and cut into runs that hand the state over through
    slots (also a slot used again by another sequence)."""
    say("op decay_scan", device)
    torch.manual_seed(1)
    for (H, N, P, G) in [(3, 8, 16, 3), (4, 6, 8, 2), (2, 48, 64, 1), (5, 1, 3, 5), (2, 130, 70, 2)]:
        n, d = 29, 12
        h = torch.randn(n, d).double()
        # --- channel gate (gated linear attention without its norm / gate / output projection)
        Wg = {"q": torch.randn(H * N, d), "k": torch.randn(H * N, d), "v": torch.randn(H * P, d), "a1": torch.randn(4, d),
              "a2": torch.randn(H * N, 4), "a2.b": torch.randn(H * N) + 2}
        Wg = {k: v.double() for k, v in Wg.items()}
        q, k, v = h @ Wg["q"].T, h @ Wg["k"].T, h @ Wg["v"].T
        zz = (h @ Wg["a1"].T) @ Wg["a2"].T
        alpha = torch.sigmoid(zz + Wg["a2.b"]).pow(1 / 3.0).view(n, H, N)
        S = torch.zeros(H, N, P).double()
        want = torch.zeros(n, H, P).double()
        for t in range(n):
            S = alpha[t][:, :, None] * S + k[t].view(H, N)[:, :, None] * v[t].view(H, P)[:, None, :]
            want[t] = torch.einsum("hnp,hn->hp", S, q[t].view(H, N) * N ** -0.5)
        for cuts in ([n], [1, 2, 9, 1, 16]):
            state = torch.randn(3, H, N, P)          # garbage: a fresh run must not read it
            out = torch.empty(n, H * P)
            slot, r0 = 1, 0
            for c in cuts:
                prev = torch.tensor([(-1 if r0 == 0 else -(slot + 2))] + list(range(c - 1)), dtype=torch.int32)
                save = torch.tensor([-1] * (c - 1) + [slot], dtype=torch.int32)
                cu = torch.tensor([0, c], dtype=torch.int32)
                a = _dev(device, q[r0:r0 + c].float(), k[r0:r0 + c].float(), v[r0:r0 + c].float(), zz[r0:r0 + c].float(),
                         Wg["a2.b"].float(), state, cu, prev, save, torch.empty(c, H * P))
                ops.decay_scan(ops.DECAY_CHANNEL_GATE, a[0], a[1], a[2], a[3], a[4], 3.0, None, N ** -0.5, H, N, P, 1, a[5],
                               a[6] if c > 1 else None, a[7], a[8], 1, a[9])
                state = a[5]
                out[r0:r0 + c] = a[9].cpu()
                r0 += c
            assert torch.allclose(out, want.reshape(n, -1).float(), atol=3e-4, rtol=3e-4), ("gate", H, N, P, cuts)
        # --- step size (state-space recurrence with groups and a skip term)
        B, Cc, x = torch.randn(n, G, N).double(), torch.randn(n, G, N).double(), torch.randn(n, H, P).double()
        dt_in, dt_b, A_log, D = torch.randn(n, H).double(), torch.randn(H).double(), torch.randn(H).double() - 1, torch.randn(H).double()
        dt = torch.nn.functional.softplus(dt_in + dt_b)
        S = torch.zeros(H, N, P).double()
        want = torch.zeros(n, H, P).double()
        for t in range(n):
            for hd in range(H):
                g = hd // (H // G)
                S[hd] = torch.exp(-torch.exp(A_log[hd]) * dt[t, hd]) * S[hd] + dt[t, hd] * B[t, g][:, None] * x[t, hd][None, :]
                want[t, hd] = S[hd].T @ Cc[t, g] + D[hd] * x[t, hd]
        state = torch.randn(2, H, N, P)
        prev = torch.tensor([-1] + list(range(n - 1)), dtype=torch.int32)
        save = torch.tensor([-1] * (n - 1) + [0], dtype=torch.int32)
        a = _dev(device, Cc.reshape(n, -1).float(), B.reshape(n, -1).float(), x.reshape(n, -1).float(), dt_in.float(),
                 dt_b.float(), A_log.float(), D.float(), state, torch.tensor([0, n], dtype=torch.int32), prev, save,
                 torch.empty(n, H * P))
        ops.decay_scan(ops.DECAY_STEP_SIZE, a[0], a[1], a[2], a[3], a[4], a[5], a[6], 1.0, H, N, P, H // G, a[7], a[8], a[9],
                       a[10], 1, a[11])
        assert torch.allclose(a[11].cpu(), want.reshape(n, -1).float(), atol=3e-4, rtol=3e-4), ("step", H, N, P)
        assert torch.allclose(a[7].cpu()[0], S.float(), atol=3e-4, rtol=3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_conv_norm_router_ops(device):
    """causal_conv_silu + conv_state_update over cut runs, gated_group_norm in both orders, softmax_topk with a
    correction that changes the choice but not the weights, moe_mix with identity experts."""
    say("op conv/norm/router", device)
    torch.manual_seed(2)
    # convolution: whole against cut into runs of 1 / 2 / many rows, taps from 1 to 5
    for taps, Cn in [(4, 11), (2, 300), (5, 7), (1, 4)]:
        n = 23
        x, w, b = torch.randn(n, Cn), torch.randn(Cn, taps), torch.randn(Cn)
        want = O.silu(O.causal_conv(x.double(), w.double(), b.double())).float()
        state = torch.randn(2, taps - 1, Cn)
        out, r0 = torch.empty(n, Cn), 0
        for c in (1, 1, 2, 1, 7, 3, 8):
            prev = torch.tensor([(-1 if r0 == 0 else -(1 + 2))] + list(range(c - 1)), dtype=torch.int32)
            save = torch.tensor([-1] * (c - 1) + [1], dtype=torch.int32)
            cu = torch.tensor([0, c], dtype=torch.int32)
            a = _dev(device, x[r0:r0 + c].contiguous(), w, b, state, cu, torch.zeros(c, dtype=torch.int32), prev, save,
                     torch.empty(c, Cn))
            ops.causal_conv_silu(a[0], a[1], a[2], a[3], a[4], a[5], a[6], 1, a[8])
            ops.conv_state_update(a[0], a[3], a[4], a[6], a[7], 1)
            state = a[3]
            out[r0:r0 + c] = a[8].cpu()
            r0 += c
        assert torch.allclose(out, want, atol=1e-4, rtol=1e-4), taps
    # gated group norm
    for Cn, group, wlen, first in [(24, 8, 8, False), (24, 12, 24, True), (600, 300, 600, True), (5, 5, 5, False)]:
        y, g, w = torch.randn(9, Cn), torch.randn(9, Cn + 3), torch.rand(wlen) + 0.5
        s = O.silu(g[:, 3:].double())
        v = (y.double() * s) if first else y.double()
        v = O.unit_rms(v.view(9, Cn // group, group), 1e-5).reshape(9, Cn) * w.double().repeat(Cn // wlen)
        want = (v if first else v * s).float()
        a = _dev(device, y, g, w, torch.empty(9, Cn))
        ops.gated_group_norm(a[0], a[1][:, 3:], a[2], 1e-5, group, first, a[3])
        assert torch.allclose(a[3].cpu(), want, atol=1e-4, rtol=1e-4), (Cn, group)
    # router: the correction lifts entry 6 into the choice; its weight stays its softmax score
    for En, k in [(7, 2), (70, 3), (1, 1), (9, 9)]:
        x, Wr = torch.randn(13, 10), torch.randn(En, 10)
        corr = torch.zeros(En)
        corr[min(6, En - 1)] = 5.0
        ids, wt = torch.zeros(13 * k, dtype=torch.int32), torch.zeros(13 * k)
        a = _dev(device, x, Wr, corr, ids, wt)
        ops.softmax_topk(a[0], a[1], a[2], k, a[3], a[4])
        idx, want_w, _ = O.route({"router": Wr.double(), "correction": corr.double()}, "", {"router": {"top": k}}, x.double())
        assert a[3].cpu().view(13, k).tolist() == idx.tolist()
        assert torch.allclose(a[4].cpu().view(13, k), want_w.float(), atol=1e-5)
    # mix: two assignments per token, ids >= E are identity experts
    T_, d, k, E = 6, 10, 2, 3
    y, h, sh, sg = torch.randn(T_ * k, d), torch.randn(T_, d), torch.randn(T_, d), torch.randn(T_, 4)
    ids = torch.tensor([0, 3, 4, 1, 2, 2, 3, 4, 1, 0, 4, 0], dtype=torch.int32)
    dst = torch.randperm(T_ * k).int()
    wt = torch.rand(T_ * k)
    want = torch.zeros(T_, d)
    for t in range(T_):
        for j in range(k):
            a_ = t * k + j
            want[t] += wt[a_] * (h[t] if ids[a_] >= E else y[dst[a_]])
        want[t] += torch.sigmoid(sg[t, 2]) * sh[t]
    a = _dev(device, y, dst, ids, wt, h, sh, sg, torch.empty(T_, d))
    ops.moe_mix(a[0], a[1], a[2], a[3], k, E, a[4], a[5], a[6][:, 2:3], a[7])
    assert torch.allclose(a[7].cpu(), want, atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_row_ops_few_wide_rows(device):
    """embed_norm, rms_norm_rows, residual_mix_norm and gated_group_norm on a handful of wide rows (the shape of a decode
    step at real widths, where the kernels use their widest workgroups) and on many narrow ones."""
    say("op rows wide", device)
    torch.manual_seed(4)
    for rows, d in [(3, 1536), (600, 40), (5, 2050)]:
        eps = 1e-5
        table, w = torch.randn(50, d), torch.randn(d) * 0.1
        ids = torch.randint(0, 50, (rows,), dtype=torch.int32)
        x = torch.empty(rows, d)
        a = _dev(device, ids, table, w, x)
        ops.embed_norm(a[0], a[1], a[2], eps, 1.0, a[3])
        want_x = O.offset_norm(table[ids.long()].double(), w.double(), eps)
        assert torch.allclose(a[3].cpu(), want_x.float(), atol=1e-5, rtol=1e-5)
        pick = torch.tensor([rows - 1, 0], dtype=torch.int64)
        out = torch.empty(2, d)
        b = _dev(device, pick, out)
        ops.rms_norm_rows(a[3], b[0], a[2], eps, 1.0, b[1])
        assert torch.allclose(b[1].cpu(), O.offset_norm(want_x[pick], w.double(), eps).float(), atol=1e-5, rtol=1e-5)
        p1, p2, p3, bias = torch.randn(rows, d), torch.randn(rows, d), torch.randn(rows, d), torch.randn(d)
        h = torch.empty(rows, d)
        c = _dev(device, p1, bias, p2, p3, h)
        ops.residual_mix_norm(a[3], c[0], 0.6, c[1], c[2], -0.5, c[3], 1.0, a[2], eps, 1.0, c[4])
        want2 = want_x + 0.6 * (p1.double() + bias.double()) - 0.5 * p2.double() + p3.double()
        assert torch.allclose(a[3].cpu(), want2.float(), atol=1e-5, rtol=1e-5)
        assert torch.allclose(c[4].cpu(), O.offset_norm(want2, w.double(), eps).float(), atol=1e-5, rtol=1e-5)
        y, g, gw = torch.randn(rows, d), torch.randn(rows, d), torch.rand(d) + 0.5
        s = O.silu(g.double())
        want3 = (O.unit_rms(y.double() * s, eps) * gw.double()).float()
        e = _dev(device, y, g, gw, torch.empty(rows, d))
        ops.gated_group_norm(e[0], e[1], e[2], eps, d, True, e[3])
        assert torch.allclose(e[3].cpu(), want3, atol=1e-5, rtol=1e-4)
