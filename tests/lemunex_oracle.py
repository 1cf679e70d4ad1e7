"""Plain, slow whole-sequence implementation of the Lemunex design: one function per mechanism, float64, no code
shared with the product path (symmetry_amd/models/lemunex.py and its kernels).

Notation: ``W`` maps name -> tensor ([out, in] matrices), ``cfg`` is the config.json dictionary, a sequence is a
[n, width] matrix with one row per token, positions 0..n-1.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


# ---- rotary ----------------------------------------------------------------------------------------------------
def rotary_frequencies(rot: dict):
    """Per pair i < dims / 2: the angular step per position, and the factor on cos / sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    i = torch.arange(dims // 2, dtype=F64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, rot: dict):
    """x [n, heads, dim]: the first rot.dims entries of every head turn, entry 2i with entry 2i + 1."""
    dims = int(rot["dims"])
    f, mag = rotary_frequencies(rot)
    ang = positions.to(F64)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---- the two halves of the 'parallel' mixer ------------------------------------------------------------------
def window_attention(W, p, spec, h):
    """Softmax attention with grouped key/value heads, a sliding window, partial rotary and a per-head sigmoid gate."""
    n = h.shape[0]
    H, G, dk, dv = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    pos = torch.arange(n)
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(n, H, dk)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(n, G, dk)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(n, G, dv)
    q, k = rotate_pairs(q, pos, spec["rot"]), rotate_pairs(k, pos, spec["rot"])
    gate = torch.sigmoid(h @ W[p + "g"].T)                       # [n, H]
    span = int(spec["mask"]["size"])
    out = torch.zeros(n, H, dv, dtype=F64)
    for t in range(n):
        j0 = max(0, t - span + 1)
        for hd in range(H):
            g = hd // (H // G)
            sc = (k[j0:t + 1, g] @ q[t, hd]) * float(spec["scale"])
            out[t, hd] = torch.softmax(sc, 0) @ v[j0:t + 1, g]
    out = out * gate[:, :, None]
    return out.reshape(n, H * dv) @ W[p + "o"].T + W[p + "o.b"]


def gated_linear_attention(W, p, spec, h, eps):
    """Per head S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t; alpha per key channel."""
    n = h.shape[0]
    H, dk, dv = spec["heads"], spec["dim"], spec["vdim"]
    q = (h @ W[p + "q"].T).view(n, H, dk) * dk ** -0.5
    k = (h @ W[p + "k"].T).view(n, H, dk)
    v = (h @ W[p + "v"].T).view(n, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / float(spec["tau"])).view(n, H, dk)
    S = torch.zeros(H, dk, dv, dtype=F64)
    o = torch.zeros(n, H, dv, dtype=F64)
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = unit_rms(o, eps) * W[p + "norm"]
    return (o.reshape(n, H * dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def parallel_mixer(W, p, spec, h, eps):
    left = window_attention(W, p + "left.", spec["left"], h)
    right = gated_linear_attention(W, p + "right.", spec["right"], h, eps)
    return float(spec["left_scale"]) * left + float(spec["right_scale"]) * right


# ---- the state-space mixer -----------------------------------------------------------------------------------
def causal_conv(x, w, b):
    """x [n, C], w [C, taps]: y_t = b + sum_j w[:, taps - 1 - j] * x_(t - j), zeros before the sequence."""
    n, taps = x.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], 0)
    y = b[None, :].expand(n, -1).clone()
    for j in range(taps):
        y = y + pad[taps - 1 - j: taps - 1 - j + n] * w[:, taps - 1 - j]
    return y


def mamba2_mixer(W, p, spec, h, eps):
    n = h.shape[0]
    Hh, P, N, G = spec["heads"], spec["vdim"], spec["state"], spec["groups"]
    inner = Hh * P
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(n, Hh, P)
    B = xbc[:, inner:inner + G * N].view(n, G, N)
    C = xbc[:, inner + G * N:].view(n, G, N)
    dt = torch.nn.functional.softplus(dt + W[p + "dt_bias"], beta=1.0, threshold=1e9)
    rate = torch.exp(W[p + "A_log"])
    S = torch.zeros(Hh, N, P, dtype=F64)
    y = torch.zeros(n, Hh, P, dtype=F64)
    for t in range(n):
        for hd in range(Hh):
            g = hd // (Hh // G)
            S[hd] = torch.exp(-rate[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * B[t, g][:, None] * x[t, hd][None, :]
            y[t, hd] = S[hd].T @ C[t, g] + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    parts = int(spec["norm_groups"])
    y = unit_rms(y.view(n, parts, inner // parts), eps).reshape(n, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


# ---- feed-forward ----------------------------------------------------------------------------------------------
def relu2_ff(W, p, h):
    return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T


def gated_expert(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(W, p, spec, h):
    """(chosen experts [n, top], their weights [n, top], margin between the last chosen and the first rejected)."""
    r = spec["router"]
    s = torch.softmax(h @ W[p + "router"].T, -1)
    pick = s + W[p + "correction"]
    order = torch.argsort(pick, dim=-1, descending=True, stable=True)
    top = int(r["top"])
    idx = order[:, :top]
    srt = torch.gather(pick, 1, order)
    margin = (srt[:, top - 1] - srt[:, top]) if srt.shape[1] > top else torch.full((h.shape[0],), math.inf, dtype=F64)
    return idx, torch.gather(s, 1, idx), margin


def moe_ff(W, p, spec, h, margins=None):
    r = spec["router"]
    E = int(r["experts"])
    idx, wt, margin = route(W, p, spec, h)
    if margins is not None:   # a near-tie only matters if the expert it may swap in or out carries weight
        margins.append(torch.where(wt[:, -1] > 0.05, margin, torch.full_like(margin, math.inf)))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wt[t]):
            out[t] += w * (h[t] if e >= E else gated_expert(W, f"{p}e{e}.", h[t:t + 1])[0])
    if spec.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * gated_expert(W, p + "shared.", h)
    return out


# ---- the model -------------------------------------------------------------------------------------------------
def forward(cfg: dict, W: dict, tokens, trace=None, margins=None):
    """Logits [n, vocab] of one sequence; ``trace`` (a list) receives the stream after every layer."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    x = offset_norm(W["embed"][torch.as_tensor(tokens)], W["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_norm(x, W[p + "norm1"], eps)
        if layer["type"] == "parallel":
            d = parallel_mixer(W, p + "mix.", layer["mixer"], h, eps)
        elif layer["type"] == "mamba2":
            d = mamba2_mixer(W, p + "mix.", layer["mixer"], h, eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            d = d + (relu2_ff(W, p + "mlp.", h) if mlp["kind"] == "dense" else moe_ff(W, p + "mlp.", mlp, h, margins))
        x = x + d
        if trace is not None:
            trace.append(x.clone())
    return offset_norm(x, W["final.norm"], eps) @ W["head"].T
