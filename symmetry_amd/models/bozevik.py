"""Bozevik decoder forward on the symmetry_amd ops: one code path for CPU (torch references) and MI355X (HIP).

The design, in this file's notation (x: the fp32 stream, one row per token; W stored [out, in])::

    x_0 = E[token]                                      X_0 = x_0 (layer history)
    per layer i:
      h   = x + (x_prev - x) * mu_i                     token shift; x_prev = the sequence's previous row of x
      a   = mixer_i(h)                                  latent attention (below)
      x   = x + LN(a) * g1_i                            layer norm on the sublayer's OUTPUT (weight, no bias)
      x   = x + LN(ff_i(x)) * g2_i                      clamped GLU, dense or routed
      X_(i+1) = x;  x = sum_{j <= i+1} dwa_i[j] X_j     depth-weighted average feeds the next layer
    logits = logit_scale * E . (LN(x) * g_f)

    mixer (H heads; per head dn unrotated + rot rotated query/key dims, dv value dims; latent ranks rq, r):
      c_q = RMS(W_dq h) * g_q            q = W_uq c_q = [q_n | q_r] per head, q_r rotated (interleaved pairs)
      [c' | k'] = W_dkv h                c = RMS(c') * g_kv, k_r = rotary(k')      -- the cache row [c | k_r]
      score_h(t, j) = scale * (q_n . W_uk,h c_j + q_r . k_r,j),  causal softmax,  out_h = W_uv,h sum_j p_j c_j
    evaluated with the up-projections folded into the query / output (ops.latent_attn): the per-head batched
    products q_n W_uk,h and (sum p c) W_uv,h^T are library bmm calls on strided views, the attention itself is
    multi-query over the paged latent cache.  A layer with ``kv_from`` = j has no W_dkv and attends layer j's plane.

Step launches per layer: token_shift, GEMM [W_dq; W_dkv], latent_prep (both RMS norms + rotary + paged cache write),
GEMM W_uq, bmm (absorb W_uk), rope_pairs, latent_attn, bmm (W_uv), GEMM W_o, add_layer_norm (+ carried-state save),
feed-forward (GEMM gate|up, clamped_glu, GEMM down; routed: sigmoid_topk, expert_offsets, scatter_scaled, grouped
gate|up, clamped_glu, grouped down, shared expert, gather_sum), add_layer_norm (+ history append + depth mix).
All intermediates live in the preallocated Workspace, so decode steps are hipGraph-capturable.

Activations are bf16 (serving) or fp32 (``dtype=torch.float32``: every product in true 32-bit, the sharper numerical
check); the stream, the layer history, the carried state, norm statistics, rotary angles, router scores, attention
scores / weights and all accumulations are fp32 in both.
"""
from __future__ import annotations

import math

import torch

from .. import ops
from .config import BozevikConfig, GluSpec, MoeSpec
from .transformer import MAX_STEP_SEQS, ForwardBatch, Workspace
from .weights import ModelWeights

GLU_ALPHA = 1.702  # slope of the gate's sigmoid (fixed by the design)


class LatentKVCache:
    """Paged latent cache + per-sequence carried state.

    ``kv``: one plane [NB, BS, r + rot] per layer that owns a down-projection (layers that attend another layer's
    latents have none), a row = normalised latent | rotated shared key part; planes may differ in width (every
    layer names its own sizes) and share the block numbering, so one BlockManager and one block table serve all.
    Zero-initialised: every byte is finite, so rows of padded batch entries (block 0) contribute finite scores.
    ``state`` [slots, L, d] fp32: per live sequence and layer, the layer input row of the sequence's newest token
    (what the next step's token shift reads as x_prev).  Slots are handed out by the scheduler's StateSlotManager.
    """

    def __init__(self, cfg: BozevikConfig, num_blocks: int, block_size: int, num_slots: int, device, dtype):
        owners = cfg.cache_layers()
        self.plane = {layer: p for p, layer in enumerate(owners)}
        self.num_layers, self.num_blocks, self.block_size = cfg.num_layers, num_blocks, block_size
        self.kv = [torch.zeros(num_blocks, block_size, cfg.layers[i].mixer.kv_rank + cfg.layers[i].mixer.rot_dim,
                               device=device, dtype=dtype) for i in owners]
        self.state = torch.zeros(num_slots, cfg.num_layers, cfg.hidden_size, device=device, dtype=torch.float32)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv) + self.state.numel() * 4


class BozevikLM:
    has_seq_state = True      # the engine allots a state slot per live sequence and sends prev_row / save_slot / row_seq
    fused = False
    single_copy = False
    moe = None
    tp = None

    def __init__(self, weights: ModelWeights, device, tp_comm=None, ep_comm=None, max_decode_ctx: int | None = None,
                 decode_weights: str = "auto", kv_reserve_bytes: int = 0, dtype=torch.bfloat16):
        if weights.shard.tp_size > 1 or weights.shard.ep_size > 1:
            raise NotImplementedError("Bozevik runs on one GPU per replica")
        self.cfg: BozevikConfig = weights.cfg
        self.w = weights
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp_size, self.tp_rank = 1, 0
        self.ws = Workspace()
        self.last_ids = torch.zeros(MAX_STEP_SEQS, dtype=torch.int32, device=self.device)
        self.last_logits = None
        cfg = self.cfg
        max_pos = min(cfg.max_position, max_decode_ctx or cfg.max_position)
        self._rope: dict = {}
        self.L = [self._prepare_layer(i, max_pos) for i in range(cfg.num_layers)]
        self.embed = weights["embed"].to(dtype)
        self.final_norm = weights["final.norm"].to(dtype)

    # ------------------------------------------------------------------------------------------
    def make_cache(self, num_blocks: int, block_size: int, num_slots: int) -> LatentKVCache:
        return LatentKVCache(self.cfg, num_blocks, block_size, num_slots, self.device, self.dtype)

    def extra_weight_bytes(self) -> int:
        return 0

    def _rope_table(self, m, max_pos: int) -> torch.Tensor:
        """[max_pos, rot_dim / 2, 2] (cos, sin): pairs past rot.dims / 2 are the identity (they pass unchanged)."""
        key = (m.rot_dim, m.rot_dims, m.rot_base, max_pos)
        if key not in self._rope:
            t = torch.zeros(max_pos, m.rot_dim // 2, 2, dtype=torch.float32)
            t[..., 0] = 1.0
            t[:, : m.rot_dims // 2] = ops.rope_pair_table(max_pos, m.rot_dims, m.rot_base)
            self._rope[key] = t.to(self.device)
        return self._rope[key]

    def _prepare_layer(self, i: int, max_pos: int) -> dict:
        """The fused / reshaped tensors layer i's launches read."""
        w, layer, dt = self.w, self.cfg.layers[i], self.dtype
        m = layer.mixer
        if m.rot_dim % 2:
            raise ValueError(f"layer {i}: rot_dim must be even")
        if m.kv_rank > 512:
            raise NotImplementedError(f"layer {i}: kv_rank {m.kv_rank} > 512 (latent_attn's accumulator registers)")
        p = f"l{i}."

        def t(name):
            return w[p + name].to(dt)

        def glu(prefix):
            return {"w_gu": torch.cat([t(prefix + "gate"), t(prefix + "up")], 0).contiguous(), "w_down": t(prefix + "down")}

        owner = m.kv_from is None
        out = {
            "mixer": m, "mlp": layer.mlp, "owner": owner, "plane_of": i if owner else m.kv_from,
            "shift": t("shift"), "norm1": t("norm1"), "norm2": t("norm2"), "dwa": w[p + "dwa"].float().contiguous(),
            "w_in": (torch.cat([t("mix.dq"), t("mix.dkv")], 0).contiguous() if owner else t("mix.dq")),
            "gq": t("mix.dq.norm"), "gkv": t("mix.dkv.norm") if owner else None,
            "uq": t("mix.uq"),
            "uk": t("mix.uk").view(m.heads, m.dim, m.kv_rank),                     # [H, dn, r]: q_n @ uk[h]
            "uvt": t("mix.uv").view(m.heads, m.vdim, m.kv_rank).transpose(1, 2),   # [H, r, dv] view
            "o": t("mix.o"), "rope": self._rope_table(m, max_pos),
        }
        if isinstance(layer.mlp, GluSpec):
            out["ff"] = glu("mlp.")
        elif isinstance(layer.mlp, MoeSpec):
            E = layer.mlp.experts
            out["router"] = t("mlp.router")
            out["w13"] = torch.stack([torch.cat([t(f"mlp.e{e}.gate"), t(f"mlp.e{e}.up")], 0) for e in range(E)]).contiguous()
            out["w2"] = torch.stack([t(f"mlp.e{e}.down") for e in range(E)]).contiguous()
            out["shared"] = glu("mlp.shared.") if layer.mlp.shared else None
        return out

    # ------------------------------------------------------------------------------------------
    def _buf(self, name, shape, dtype=None):
        return self.ws.get(name, shape, dtype or self.dtype, self.device)

    def _linear(self, name: str, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x [R, K] @ w[N, K]^T -> [R, N] in the activation dtype (library GEMM, fp32 accumulation)."""
        return ops.linear(x, w, out=self._buf(name, (x.shape[0], w.shape[0])))

    def _glu(self, name: str, x: torch.Tensor, f: dict, spec: GluSpec) -> torch.Tensor:
        gu = self._linear(name + ".gu", x, f["w_gu"])
        act = self._buf(name + ".act", (x.shape[0], spec.ff))
        ops.clamped_glu(gu, spec.limit, GLU_ALPHA, act)
        return self._linear(name + ".down", act, f["w_down"])

    def _grouped(self, xs: torch.Tensor, W: torch.Tensor, offsets: torch.Tensor, y: torch.Tensor) -> None:
        """y = xs @ W[e]^T over the expert segments: the main kernel library's MFMA grouped GEMM (bf16, shapes that
        tile for it: K % 64, N % 128, at most 64 experts) where that library is built, else the all-shapes kernel."""
        E, N, K = W.shape
        if (self.dtype == torch.bfloat16 and self.device.type != "cpu" and not ops.torch_mode() and E <= 64
                and K % 64 == 0 and N % 128 == 0 and ops.native_available()):
            ops.grouped_gemm(xs, W, offsets, 0, y, ops.GROUPED_BF16)
        else:
            ops.grouped_linear(xs, W, offsets, y)

    def _moe(self, P: dict, x: torch.Tensor) -> torch.Tensor:
        """Routed feed-forward: fp32 sigmoid scores, top-k, each chosen expert applied to (score * x), plus the shared
        expert; returns the fp32 sum.  Segment bounds stay on the device (no host sync: graph-capturable)."""
        spec: MoeSpec = P["mlp"]
        T, d = x.shape
        E, k = spec.experts, spec.top
        R = T * k
        i32 = torch.int32
        ids, wts = self._buf("moe.ids", (R,), i32), self._buf("moe.w", (R,), torch.float32)
        offsets, cursor = self._buf("moe.offsets", (E + 1,), i32), self._buf("moe.cursor", (E,), i32)
        dst = self._buf("moe.dst", (R,), i32)
        xs = self._buf("moe.xs", (R, d))
        ops.sigmoid_topk(x, P["router"], k, ids, wts)
        ops.expert_offsets(ids, R, E, offsets, cursor)
        ops.scatter_scaled(x, ids, wts, k, offsets, cursor, xs, dst)
        F = spec.expert.ff
        y1 = self._buf("moe.y1", (R, 2 * F))
        self._grouped(xs, P["w13"], offsets, y1)
        act = self._buf("moe.act", (R, F))
        ops.clamped_glu(y1, spec.expert.limit, GLU_ALPHA, act)
        y2 = self._buf("moe.y2", (R, d))
        self._grouped(act, P["w2"], offsets, y2)
        shared = self._glu("moe.shared", x, P["shared"], spec.shared) if P["shared"] is not None else None
        out = self._buf("moe.out", (T, d), torch.float32)
        ops.gather_sum(y2, dst, k, shared, out)
        return out

    def _mixer(self, P: dict, b: ForwardBatch, cache: LatentKVCache, h: torch.Tensor) -> torch.Tensor:
        m = P["mixer"]
        T, H, r, rot, dn = h.shape[0], m.heads, m.kv_rank, m.rot_dim, m.dim
        eps = self.cfg.norm_eps
        plane = cache.kv[cache.plane[P["plane_of"]]]
        z = self._linear("z", h, P["w_in"])
        cq = self._buf("cq", (T, m.q_rank))
        ops.latent_prep(z, m.q_rank, r if P["owner"] else 0, rot, P["gq"], P["gkv"], eps, b.positions, b.slot_mapping,
                        P["rope"], cq, plane if P["owner"] else None)
        q = self._linear("q", cq, P["uq"]).view(T, H, dn + rot)
        qa = self._buf("qa", (T, H, r + rot))
        torch.bmm(q[:, :, :dn].transpose(0, 1), P["uk"], out=qa[:, :, :r].transpose(0, 1))
        ops.rope_pairs(q[:, :, dn:], qa[:, :, r:], b.positions, P["rope"])
        olat = self._buf("olat", (T, H, r))
        part_o = part_ml = None
        if b.kind == "decode" and self.device.type != "cpu":
            parts = ops.latent_attn_parts(T, b.block_tables.shape[1] * cache.block_size)
            if parts > 1:
                part_o = self._buf("attn.part_o", (T, H, parts, r), torch.float32)
                part_ml = self._buf("attn.part_ml", (T, H, parts, 2), torch.float32)
        tiled = b.kind != "decode" and self.dtype == torch.bfloat16
        ops.latent_attn(qa, plane, b.block_tables, b.row_seq, b.positions, m.scale, r, olat, part_o, part_ml,
                        b.tiles if tiled else None, b.cu_q if tiled else None)
        ov = self._buf("ov", (T, H * m.vdim))
        torch.bmm(olat.transpose(0, 1), P["uvt"], out=ov.view(T, H, m.vdim).transpose(0, 1))
        return self._linear("att", ov, P["o"])

    @torch.no_grad()
    def forward(self, b: ForwardBatch, cache: LatentKVCache) -> torch.Tensor:
        """Run one step; returns sampled token ids [num_seqs] int32 (device).  ``b.logit_rows`` (prefill-kind steps)
        or ``b.need_logits`` (decode steps: every row) leave fp32 logits in ``self.last_logits``."""
        cfg = self.cfg
        T, d, eps, nl = b.num_tokens, cfg.hidden_size, cfg.norm_eps, cfg.num_layers
        f32 = torch.float32
        x = self._buf("x", (T, d), f32)
        hist = self._buf("hist", (nl + 1, T, d), f32)
        h = self._buf("h", (T, d))
        src = b.src if b.src is not None and b.kind == "decode" else None
        ops.embed_rows(b.input_ids, self.embed, x, hist[0], src, self.last_ids if src is not None else None)
        for i, P in enumerate(self.L):
            st = cache.state[:, i]
            ops.token_shift(x, P["shift"], b.prev_row, st, h)
            att = self._mixer(P, b, cache, h)
            if P["mlp"] is None:
                ops.add_layer_norm(att, P["norm1"], eps, x, b.save_slot, st, hist, P["dwa"], i + 1, None)
                continue
            xa = self._buf("xa", (T, d))
            ops.add_layer_norm(att, P["norm1"], eps, x, b.save_slot, st, None, None, 0, xa)
            delta = self._moe(P, xa) if isinstance(P["mlp"], MoeSpec) else self._glu("ff", xa, P["ff"], P["mlp"])
            ops.add_layer_norm(delta, P["norm2"], eps, x, None, None, hist, P["dwa"], i + 1, None)
        n = b.num_seqs
        ids = self.last_ids[:n]
        self.last_logits = None
        if b.sample or b.need_logits:
            rows = None if b.kind == "decode" else b.last_idx
            logits = self._logits("logits", x, rows, n)
            if b.need_logits:
                self.last_logits = logits
            if b.sample:
                keys = self._buf("keys", (n,), torch.int64)
                ops.logits_argmax(logits, b.temps, b.seeds, b.step, keys, ids, 0)
                if b.filtered:
                    ops.sample_filtered(logits, b.temps, b.top_k, b.top_p, b.seeds, b.step, ids)
        if b.logit_rows is not None and b.logit_rows.numel():
            self.last_logits = self._logits("want_logits", x, b.logit_rows, int(b.logit_rows.numel()))
        return ids

    def _logits(self, name: str, x: torch.Tensor, rows, n: int) -> torch.Tensor:
        """fp32 logits [n, V] = logit_scale * LN(x[rows]) . E^T (fp32 output from the library GEMM)."""
        cfg = self.cfg
        xn = self._buf(name + ".xn", (n, cfg.hidden_size))
        ops.layer_norm(x, rows, self.final_norm, cfg.norm_eps, xn)
        logits = self._buf(name, (n, cfg.vocab_size), torch.float32)
        if self.dtype == torch.float32:
            torch.matmul(xn, self.embed.t(), out=logits)
        elif self.device.type == "cpu":
            logits.copy_(xn.float() @ self.embed.float().t())
        else:
            torch.bmm(xn[None], self.embed.t()[None], out_dtype=torch.float32, out=logits[None])
        if cfg.logit_scale != 1.0:
            logits.mul_(cfg.logit_scale)
        return logits
