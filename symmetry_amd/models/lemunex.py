"""Lemunex decoder forward on the symmetry_amd ops: one code path for CPU (torch references) and MI355X (HIP).

The design, in this file's notation (x: the fp32 stream, one row per token; W stored [out, in]; n(v, g) =
v / sqrt(mean(v^2) + eps) * (1 + g))::

    x = n(E[token], g_e)
    per layer i:   h = n(x, g_i);   x = x + mixer_i(h) + ff_i(h)         (one norm feeds both sublayers)
    logits = W_head n(x, g_f)

    mixer "parallel" = c_l * A(h) + c_r * R(h), both reading h:
      A: q, k, v = W h + b; q, k turned by the scaled rotary on their first rot.dims entries (interleaved pairs);
         softmax over the positions p - window < j <= p; query head h reads key / value head h // (H / G);
         head outputs times sigmoid(W_g h)_h; W_o (.) + b_o
      R: per head S <- diag(a_t) S + k_t v_t^T, o_t = S^T q_t / sqrt(dim), a = sigmoid(W_a2 W_a1 h + b_a)^(1 / tau) per
         key channel; o normalised per head (plain weight), times silu(W_g h), W_o
    mixer "mamba2": W_in h = [z | x | B | C | dt]; x, B, C through a causal per-channel convolution + silu;
         dt = softplus(dt + dt_bias); per head S <- exp(-exp(A_log) dt) S + dt B_t x_t^T, y = S^T C_t + D x_t;
         y * silu(z), RMS norm in norm_groups parts, W_o
    ff: W_down relu(W_up h)^2, or routed: s = softmax(W_r h) over experts + identity experts, the ``top`` largest of
         s + correction, output sum_e s_e expert_e(h) (identity: h itself), expert = W_down (silu(W_gate h) * W_up h),
         plus sigmoid(W_sg h) * shared(h)

Every projection that reads h is one row block of ONE fused weight per layer (a single library GEMM); the kernels take
column ranges of its output as views.  Step launches per layer: GEMM (all of h's projections), then
parallel: qkv_rope_cache, window_attn, GEMM W_o | GEMM W_a2, decay_scan, gated_group_norm, GEMM W_o
mamba2:   causal_conv_silu, conv_state_update, decay_scan, gated_group_norm, GEMM W_o
ff:       relu_sq, GEMM down | softmax_topk, expert_offsets, scatter, grouped gate|up, silu_mul, grouped down,
          silu_mul + GEMM (shared), moe_mix
and one residual_mix_norm that adds the scaled sublayer outputs to the stream and emits the next layer's h.
All intermediates live in the preallocated Workspace, so decode steps are hipGraph-capturable.

fp32 in both serving dtypes: the stream, norm statistics, rotary angles, attention scores and weights, the recurrent
states, decays / step sizes and everything derived from them, router scores.  ``dtype=torch.float32`` runs every
product in true 32-bit as well.
"""
from __future__ import annotations

import torch

from .. import ops
from .config import LemunexConfig, ReluSqSpec, RoutedSpec
from .transformer import MAX_STEP_SEQS, ForwardBatch, Workspace
from .weights import ModelWeights

NORM_OFFSET = 1.0     # stream norms store their weight as the deviation from one (fixed by the design)
SEG_ALIGN = 8         # row blocks of the fused projection start at multiples of 8 columns (16-byte bf16 accesses)


class HybridCache:
    """What a hybrid model keeps per sequence.

    ``k`` / ``v``: one pair of paged planes per attention layer, [NB, BS, G, dk] / [NB, BS, G, dv] (token-major), on
    the engine's BlockManager numbering (one block table serves all planes).  ``rec``: per recurrent layer the
    matrix state [slots, H, N, P] fp32; ``conv``: per convolution the newest taps - 1 inputs [slots, taps - 1, C].
    Slots are handed out by the scheduler's StateSlotManager; a slot's old content is never read by a new sequence
    (its first run starts from zero).  Zero-initialised: every byte finite."""

    def __init__(self, cfg: LemunexConfig, num_blocks: int, block_size: int, num_slots: int, device, dtype):
        self.num_layers, self.num_blocks, self.block_size = cfg.num_layers, num_blocks, block_size
        self.k, self.v, self.rec, self.conv = {}, {}, {}, {}
        for i, layer in enumerate(cfg.layers):
            m = layer.mixer
            if layer.type == "parallel":
                a, g = m.left, m.right
                self.k[i] = torch.zeros(num_blocks, block_size, a.kv_heads, a.dim, device=device, dtype=dtype)
                self.v[i] = torch.zeros(num_blocks, block_size, a.kv_heads, a.vdim, device=device, dtype=dtype)
                self.rec[i] = torch.zeros(num_slots, g.heads, g.dim, g.vdim, device=device, dtype=torch.float32)
            else:
                self.rec[i] = torch.zeros(num_slots, m.heads, m.state, m.vdim, device=device, dtype=torch.float32)
                self.conv[i] = torch.zeros(num_slots, m.conv - 1, m.conv_channels, device=device, dtype=dtype)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for d in (self.k, self.v, self.rec, self.conv) for t in d.values())


class _Fused:
    """Row blocks of a layer's fused input projection: name -> (first column, width) of its output."""

    def __init__(self):
        self.blocks, self.cols, self.n = [], {}, 0

    def add(self, name: str, w: torch.Tensor) -> None:
        pad = -self.n % SEG_ALIGN
        if pad:
            self.blocks.append(torch.zeros(pad, w.shape[1], dtype=w.dtype, device=w.device))
            self.n += pad
        self.cols[name] = (self.n, w.shape[0])
        self.blocks.append(w)
        self.n += w.shape[0]

    def weight(self) -> torch.Tensor:
        pad = -self.n % SEG_ALIGN
        tail = [torch.zeros(pad, self.blocks[0].shape[1], dtype=self.blocks[0].dtype, device=self.blocks[0].device)] if pad else []
        return torch.cat(self.blocks + tail, 0).contiguous()


class LemunexLM:
    has_seq_state = True      # the engine allots a state slot per live sequence and sends prev_row / save_slot / row_seq
    fused = False
    single_copy = False
    moe = None
    tp = None

    def __init__(self, weights: ModelWeights, device, tp_comm=None, ep_comm=None, max_decode_ctx: int | None = None,
                 decode_weights: str = "auto", kv_reserve_bytes: int = 0, dtype=torch.bfloat16):
        if weights.shard.tp_size > 1 or weights.shard.ep_size > 1:
            raise NotImplementedError("Lemunex runs on one GPU per replica")
        self.cfg: LemunexConfig = weights.cfg
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
        self._ones: torch.Tensor | None = None
        self.L = [self._prepare_layer(i, max_pos) for i in range(cfg.num_layers)]
        self.embed = weights["embed"].to(dtype)
        self.embed_norm = weights["embed.norm"].float()
        self.final_norm = weights["final.norm"].float()
        self.head = weights["head"].to(dtype)

    # ------------------------------------------------------------------------------------------
    def make_cache(self, num_blocks: int, block_size: int, num_slots: int) -> HybridCache:
        return HybridCache(self.cfg, num_blocks, block_size, num_slots, self.device, self.dtype)

    def extra_weight_bytes(self) -> int:
        return 0

    def _rope_table(self, rot, max_pos: int) -> torch.Tensor:
        key = (rot, max_pos)
        if key not in self._rope:
            self._rope[key] = ops.rope_scaled_table(max_pos, rot.dims, rot.base, rot.factor, rot.original, rot.fast,
                                                    rot.slow).to(self.device)
        return self._rope[key]

    def _prepare_layer(self, i: int, max_pos: int) -> dict:
        """The fused / converted tensors layer i's launches read.  Matrices in the activation dtype; norm weights,
        biases and the parameters of decays and step sizes in fp32."""
        w, layer, dt = self.w, self.cfg.layers[i], self.dtype
        p = f"l{i}."

        def t(name):
            return w[p + name].to(dt)

        def f(name):
            return w[p + name].float().contiguous()

        fz = _Fused()
        P = {"kind": layer.type, "mixer": layer.mixer, "mlp": layer.mlp, "norm1": f("norm1")}
        m = layer.mixer
        if layer.type == "parallel":
            a = m.left
            fz.add("left", torch.cat([t("mix.left.q"), t("mix.left.k"), t("mix.left.v")], 0))
            fz.add("left.g", t("mix.left.g"))
            for nm in ("q", "k", "v", "g", "a1"):
                fz.add("right." + nm, t("mix.right." + nm))
            P["left.b"] = torch.cat([f("mix.left.q.b"), f("mix.left.k.b"), f("mix.left.v.b")]).contiguous()
            P["left.o"], P["left.o.b"] = t("mix.left.o"), f("mix.left.o.b")
            P["right.a2"], P["right.a2.b"] = t("mix.right.a2"), f("mix.right.a2.b")
            P["right.norm"], P["right.o"] = f("mix.right.norm"), t("mix.right.o")
            P["rope"] = self._rope_table(a.rot, max_pos)
        else:
            win = t("mix.in")
            inner, gn = m.inner, m.groups * m.state
            fz.add("z", win[:inner])
            fz.add("xbc", win[inner:2 * inner + 2 * gn])
            fz.add("dt", win[2 * inner + 2 * gn:])
            P["conv"], P["conv.b"] = t("mix.conv").contiguous(), f("mix.conv.b")
            P["dt_bias"], P["A_log"], P["D"] = f("mix.dt_bias"), f("mix.A_log"), f("mix.D")
            P["norm"], P["o"] = f("mix.norm"), t("mix.o")
        mlp = layer.mlp
        if isinstance(mlp, ReluSqSpec):
            fz.add("up", t("mlp.up"))
            P["down"] = t("mlp.down")
        elif isinstance(mlp, RoutedSpec):
            E = mlp.experts
            P["router"], P["correction"] = t("mlp.router").contiguous(), f("mlp.correction")
            P["w13"] = torch.stack([torch.cat([t(f"mlp.e{e}.gate"), t(f"mlp.e{e}.up")], 0) for e in range(E)]).contiguous()
            P["w2"] = torch.stack([t(f"mlp.e{e}.down") for e in range(E)]).contiguous()
            if mlp.shared_ff:
                fz.add("shared.gate", t("mlp.shared.gate"))
                fz.add("shared.up", t("mlp.shared.up"))
                fz.add("shared.sg", t("mlp.shared.sg"))
                P["shared.down"] = t("mlp.shared.down")
        P["w_h"], P["cols"] = fz.weight(), fz.cols
        return P

    # ------------------------------------------------------------------------------------------
    def _buf(self, name, shape, dtype=None):
        return self.ws.get(name, shape, dtype or self.dtype, self.device)

    def _linear(self, name: str, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x [R, K] @ w[N, K]^T -> [R, N] in the activation dtype (library GEMM, fp32 accumulation)."""
        return ops.linear(x, w, out=self._buf(name, (x.shape[0], w.shape[0])))

    @staticmethod
    def _cols(z: torch.Tensor, P: dict, name: str) -> torch.Tensor:
        c0, n = P["cols"][name]
        return z[:, c0:c0 + n]

    def _grouped(self, xs: torch.Tensor, W: torch.Tensor, offsets: torch.Tensor, y: torch.Tensor) -> None:
        """y = xs @ W[e]^T over the expert segments: the main kernel library's MFMA grouped GEMM (bf16, shapes that
        tile for it: K % 64, N % 128, at most 64 experts) where that library is built, else the all-shapes kernel."""
        E, N, K = W.shape
        if (self.dtype == torch.bfloat16 and self.device.type != "cpu" and not ops.torch_mode() and E <= 64
                and K % 64 == 0 and N % 128 == 0 and ops.native_available()):
            ops.grouped_gemm(xs, W, offsets, 0, y, ops.GROUPED_BF16)
        else:
            ops.hyb_grouped_linear(xs, W, offsets, y)

    def _routed(self, P: dict, h: torch.Tensor, z: torch.Tensor) -> torch.Tensor:
        """Routed feed-forward -> fp32 [T, d].  Segment bounds stay on the device (no host sync: graph-capturable);
        identity experts get (unused) segments past the last real expert, their rows are mixed from h directly."""
        spec: RoutedSpec = P["mlp"]
        T, d = h.shape
        E, k, En = spec.experts, spec.top, spec.experts + spec.identity
        R, F = T * k, spec.expert_ff
        i32 = torch.int32
        ids, wts = self._buf("moe.ids", (R,), i32), self._buf("moe.w", (R,), torch.float32)
        offsets, cursor = self._buf("moe.offsets", (En + 1,), i32), self._buf("moe.cursor", (En,), i32)
        dst = self._buf("moe.dst", (R,), i32)
        xs = self._buf("moe.xs", (R, d))
        if self._ones is None or self._ones.numel() < R:
            self._ones = torch.ones(max(R, 4096), dtype=torch.float32, device=self.device)
        ops.softmax_topk(h, P["router"], P["correction"], k, ids, wts)
        ops.hyb_expert_offsets(ids, R, En, offsets, cursor)
        ops.hyb_scatter_scaled(h, ids, self._ones[:R], k, offsets, cursor, xs, dst)
        y1 = self._buf("moe.y1", (R, 2 * F))
        self._grouped(xs, P["w13"], offsets, y1)
        act = self._buf("moe.act", (R, F))
        ops.silu_mul(y1[:, :F], y1[:, F:], act)
        y2 = self._buf("moe.y2", (R, d))
        self._grouped(act, P["w2"], offsets, y2)
        shared = sgate = None
        if spec.shared_ff:
            sact = self._buf("moe.sact", (T, spec.shared_ff))
            ops.silu_mul(self._cols(z, P, "shared.gate"), self._cols(z, P, "shared.up"), sact)
            shared = self._linear("moe.shared", sact, P["shared.down"])
            sgate = self._cols(z, P, "shared.sg")
        out = self._buf("moe.out", (T, d), torch.float32)
        ops.moe_mix(y2, dst, ids, wts, k, E, h, shared, sgate, out)
        return out

    def _ff(self, P: dict, h: torch.Tensor, z: torch.Tensor):
        mlp = P["mlp"]
        if mlp is None:
            return None
        if isinstance(mlp, RoutedSpec):
            return self._routed(P, h, z)
        act = self._buf("ff.act", (h.shape[0], mlp.ff))
        ops.relu_sq(self._cols(z, P, "up"), act)
        return self._linear("ff.down", act, P["down"])

    def _pair(self, i: int, P: dict, b: ForwardBatch, cache: HybridCache, z: torch.Tensor, runs: int):
        """Both halves of a parallel mixer -> (attention output, linear-attention output), each [T, d] before its scale."""
        m = P["mixer"]
        a, g = m.left, m.right
        T = z.shape[0]
        prefill = b.kind != "decode"
        # windowed attention
        c0, n = P["cols"]["left"]
        q = self._buf("att.q", (T, a.heads, a.dim))
        ops.qkv_rope_cache(z[:, c0:c0 + n], P["left.b"], a.heads, a.kv_heads, a.dim, a.vdim, b.positions, b.slot_mapping,
                           P["rope"], q, cache.k[i], cache.v[i])
        att = self._buf("att.o", (T, a.heads, a.vdim))
        ops.window_attn(q, cache.k[i], cache.v[i], b.block_tables, b.row_seq, b.positions, a.window, a.scale,
                        self._cols(z, P, "left.g"), att, b.tiles if prefill else None, b.cu_q if prefill else None)
        left = self._linear("att.out", att.view(T, a.heads * a.vdim), P["left.o"])
        # gated linear attention
        dz = self._linear("gla.dz", self._cols(z, P, "right.a1"), P["right.a2"])
        y = self._buf("rec.y", (T, g.heads * g.vdim), torch.float32)
        ops.decay_scan(ops.DECAY_CHANNEL_GATE, self._cols(z, P, "right.q"), self._cols(z, P, "right.k"),
                       self._cols(z, P, "right.v"), dz, P["right.a2.b"], g.tau, None, g.dim ** -0.5, g.heads, g.dim,
                       g.vdim, 1, cache.rec[i], b.cu_q if prefill else None, b.prev_row, b.save_slot, runs, y)
        gy = self._buf("rec.gy", (T, g.heads * g.vdim))
        ops.gated_group_norm(y, self._cols(z, P, "right.g"), P["right.norm"], self.cfg.norm_eps, g.vdim, False, gy)
        right = self._linear("gla.out", gy, P["right.o"])
        return left, right

    def _ssm(self, i: int, P: dict, b: ForwardBatch, cache: HybridCache, z: torch.Tensor, runs: int) -> torch.Tensor:
        m = P["mixer"]
        T = z.shape[0]
        cu = b.cu_q if b.kind != "decode" else None
        xin = self._cols(z, P, "xbc")
        xc = self._buf("ssm.xc", (T, m.conv_channels))
        ops.causal_conv_silu(xin, P["conv"], P["conv.b"], cache.conv[i], cu, b.row_seq, b.prev_row, runs, xc)
        ops.conv_state_update(xin, cache.conv[i], cu, b.prev_row, b.save_slot, runs)
        inner, gn = m.inner, m.groups * m.state
        y = self._buf("rec.y", (T, inner), torch.float32)
        ops.decay_scan(ops.DECAY_STEP_SIZE, xc[:, inner + gn:], xc[:, inner:inner + gn], xc[:, :inner],
                       self._cols(z, P, "dt"), P["dt_bias"], P["A_log"], P["D"], 1.0, m.heads, m.state, m.vdim,
                       m.heads // m.groups, cache.rec[i], cu, b.prev_row, b.save_slot, runs, y)
        gy = self._buf("rec.gy", (T, inner))
        ops.gated_group_norm(y, self._cols(z, P, "z"), P["norm"], self.cfg.norm_eps, inner // m.norm_groups, True, gy)
        return self._linear("ssm.out", gy, P["o"])

    @torch.no_grad()
    def forward(self, b: ForwardBatch, cache: HybridCache) -> torch.Tensor:
        """Run one step; returns sampled token ids [num_seqs] int32 (device).  ``b.logit_rows`` (prefill-kind steps)
        or ``b.need_logits`` (decode steps: every row) leave fp32 logits in ``self.last_logits``."""
        cfg = self.cfg
        T, d, eps = b.num_tokens, cfg.hidden_size, cfg.norm_eps
        runs = b.num_seqs if b.kind != "decode" else T
        x = self._buf("x", (T, d), torch.float32)
        h = self._buf("h", (T, d))
        src = b.src if b.src is not None and b.kind == "decode" else None
        ops.embed_norm(b.input_ids, self.embed, self.embed_norm, eps, NORM_OFFSET, x, src,
                       self.last_ids if src is not None else None)
        ops.rms_norm_rows(x, None, self.L[0]["norm1"], eps, NORM_OFFSET, h)
        for i, P in enumerate(self.L):
            z = self._linear("z", h, P["w_h"])
            ff = self._ff(P, h, z)
            nxt = self.L[i + 1]["norm1"] if i + 1 < len(self.L) else None
            out = h if nxt is not None else None
            if P["kind"] == "parallel":
                left, right = self._pair(i, P, b, cache, z, runs)
                m = P["mixer"]
                ops.residual_mix_norm(x, left, m.left_scale, P["left.o.b"], right, m.right_scale, ff, 1.0, nxt, eps,
                                      NORM_OFFSET, out)
            else:
                mix = self._ssm(i, P, b, cache, z, runs)
                ops.residual_mix_norm(x, mix, 1.0, None, ff, 1.0, None, 0.0, nxt, eps, NORM_OFFSET, out)
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
        """fp32 logits [n, V] = n(x[rows], g_f) . W_head^T (fp32 output from the library GEMM)."""
        cfg = self.cfg
        xn = self._buf(name + ".xn", (n, cfg.hidden_size))
        ops.rms_norm_rows(x, rows, self.final_norm, cfg.norm_eps, NORM_OFFSET, xn)
        logits = self._buf(name, (n, cfg.vocab_size), torch.float32)
        if self.dtype == torch.float32:
            torch.matmul(xn, self.head.t(), out=logits)
        elif self.device.type == "cpu":
            logits.copy_(xn.float() @ self.head.float().t())
        else:
            torch.bmm(xn[None], self.head.t()[None], out_dtype=torch.float32, out=logits[None])
        return logits
