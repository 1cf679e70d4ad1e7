"""Plain, slow implementation of the Bozevik design, one function per mechanism, written from the design's
equations.  It shares no code with the product path (no symmetry_amd import): whole-sequence recompute,
no cache, no paging, no batching.  The tests compare the engine against it.

Notation: ``W`` matrices are stored [out, in] and applied as ``x @ W.T``; ``p`` is a dict of tensors keyed by
the checkpoint's names; ``cfg`` is the checkpoint's config.json as a dict.
"""
from __future__ import annotations

import math

import torch

GLU_ALPHA = 1.702
ROUTER_MARGINS = None  # a list: moe_ff appends, per call, the smallest gap between a token's last chosen and first
                       # rejected router logit (tests use it to keep close calls out of reduced-precision comparisons)


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def token_shift(h, mu):
    """h [T, d] -> h + (h_prev - h) * mu, h_prev the row above (zeros for the first)."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def rotate_pairs(x, pos, base, dims):
    """Interleaved rotary on the first ``dims`` entries of the last axis: (x[2i], x[2i+1]) turn by pos * base^(-2i/dims).
    x [T, ..., D], pos [T]."""
    T = x.shape[0]
    i = torch.arange(dims // 2, dtype=x.dtype)
    f = base ** (-2.0 * i / dims)
    a = pos.to(x.dtype)[:, None] * f[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_kv(p, pre, m, h, pos, eps):
    """The cached pair of a layer that owns a down-projection: latent c [T, r] and rotated shared key [T, rot]."""
    r, rot = m["kv_rank"], m["rot_dim"]
    z = h @ p[pre + "dkv"].T
    c = rms_unit(z[:, :r], eps) * p[pre + "dkv.norm"]
    kr = rotate_pairs(z[:, r:r + rot], pos, m["rot"]["base"], m["rot"]["dims"])
    return c, kr


def latent_attention(p, pre, m, h, pos, eps, c, kr):
    """Queries through a latent, keys / values from the latent (c, kr) of this or another layer; causal softmax."""
    H, dn, rot, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    cq = rms_unit(h @ p[pre + "dq"].T, eps) * p[pre + "dq.norm"]
    q = (cq @ p[pre + "uq"].T).view(T, H, dn + rot)
    qn = q[..., :dn]
    qr = rotate_pairs(q[..., dn:], pos, m["rot"]["base"], m["rot"]["dims"])
    kn = (c @ p[pre + "uk"].T).view(T, H, dn)
    v = (c @ p[pre + "uv"].T).view(T, H, dv)
    s = (torch.einsum("thd,shd->hts", qn, kn) + torch.einsum("thd,sd->hts", qr, kr)) * m["scale"]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    w = torch.softmax(s, -1)
    o = torch.einsum("hts,shd->thd", w, v).reshape(T, H * dv)
    return o @ p[pre + "o"].T


def glu_ff(p, pre, h, limit):
    g = (h @ p[pre + "gate"].T).clamp(max=limit)
    u = (h @ p[pre + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(GLU_ALPHA * g) * (u + 1)) @ p[pre + "down"].T


def moe_ff(p, pre, mlp, h):
    E, k = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ p[pre + "router"].T
    s = torch.sigmoid(z)
    top = s.topk(k, dim=-1)
    if ROUTER_MARGINS is not None and k < E:
        zs = z.sort(-1, descending=True).values
        ROUTER_MARGINS.append(float((zs[:, k - 1] - zs[:, k]).min()))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(k):
            e = int(top.indices[t, j])
            out[t] += glu_ff(p, f"{pre}e{e}.", (top.values[t, j] * h[t])[None], mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + glu_ff(p, pre + "shared.", h, mlp["shared"]["limit"])
    return out


def feed_forward(p, pre, mlp, h):
    if mlp["kind"] == "dense":
        return glu_ff(p, pre, h, mlp["limit"])
    return moe_ff(p, pre, mlp, h)


def forward(cfg, p, ids, dtype=torch.float64, trace=None):
    """Logits [T, vocab] of one sequence.  ``trace``: list that receives the stream after every layer."""
    p = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in p.items()}
    eps = cfg["norm"]["eps"]
    T = len(ids)
    pos = torch.arange(T)
    x = p["embed"][torch.tensor(ids)]
    hist = [x]
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m = L["mixer"]
        h = token_shift(x, p[pre + "shift"])
        if L["type"] != "latent_attention":
            raise ValueError(L["type"])
        if "kv_from" in m and m["kv_from"] is not None:
            c, kr = kv[m["kv_from"]]
        else:
            c, kr = kv[i] = latent_kv(p, pre + "mix.", m, h, pos, eps)
        x = x + layer_norm(latent_attention(p, pre + "mix.", m, h, pos, eps, c, kr), p[pre + "norm1"], eps)
        if L.get("mlp"):
            x = x + layer_norm(feed_forward(p, pre + "mlp.", L["mlp"], x), p[pre + "norm2"], eps)
        hist.append(x)
        d = p[pre + "dwa"]
        x = sum(d[j] * hist[j] for j in range(i + 2))
        if trace is not None:
            trace.append(x)
    x = layer_norm(x, p["final.norm"], eps)
    return (x @ p["embed"].T) * cfg["logit_scale"]


def make_config(width=64, vocab=96, layers=None, eps=1e-5, logit_scale=1.5):
    return {"architecture": "Bozevik", "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


def mixer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=24, base=10000.0, scale=None, kv_from=None):
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": {"base": base, "dims": rot_dim},
         "rot_dim": rot_dim, "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim), "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff=48, limit=1.5):
    return {"ff": ff, "kind": "dense", "limit": limit}


def moe(experts=4, top=2, ff=16, limit=2.0, shared_ff=24, shared_limit=2.5):
    d = {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared_ff:
        d["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return d


def tensor_shapes(cfg):
    d, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, d), "final.norm": (d,)}
    for i, L in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", L["mixer"]
        H, dn, rot, dv, r, rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        out[pre + "norm1"] = (d,)
        out[pre + "norm2"] = (d,)
        out[pre + "shift"] = (d,)
        out[pre + "dwa"] = (i + 2,)
        out[pre + "mix.dq"] = (rq, d)
        out[pre + "mix.dq.norm"] = (rq,)
        out[pre + "mix.uq"] = (H * (dn + rot), rq)
        if m.get("kv_from") is None:
            out[pre + "mix.dkv"] = (r + rot, d)
            out[pre + "mix.dkv.norm"] = (r,)
        out[pre + "mix.uk"] = (H * dn, r)
        out[pre + "mix.uv"] = (H * dv, r)
        out[pre + "mix.o"] = (d, H * dv)
        mlp = L.get("mlp")
        if not mlp:
            continue

        def ff(prefix, f):
            out[prefix + "gate"], out[prefix + "up"], out[prefix + "down"] = (f, d), (f, d), (d, f)

        if mlp["kind"] == "dense":
            ff(pre + "mlp.", mlp["ff"])
        else:
            for e in range(mlp["router"]["experts"]):
                ff(f"{pre}mlp.e{e}.", mlp["expert"]["ff"])
            out[pre + "mlp.router"] = (mlp["router"]["experts"], d)
            if mlp.get("shared"):
                ff(pre + "mlp.shared.", mlp["shared"]["ff"])
    return out


def random_tensors(cfg, seed=0):
    """bf16 tensors with activations of order one everywhere (so that every branch matters in the logits)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("norm") or name.endswith("norm1") or name.endswith("norm2"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
            if name.endswith("norm1") or name.endswith("norm2"):
                t = t * 0.5
        elif name.endswith("shift"):
            t = torch.rand(shape, generator=g)
        elif name.endswith("dwa"):
            t = torch.rand(shape, generator=g) * 0.5
            t[-1] += 0.75
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16)
    return out
