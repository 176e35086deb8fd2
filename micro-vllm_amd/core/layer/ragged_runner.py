"""Step function of the "ragged" model family (models/registry.py): one forward over a step's tokens -
portions of prompts beside single decoded tokens, all rows in one set of launches - reading and
extending what each sequence holds in the HybridCacheManager.  Stands beside ModelPrefillRunner /
ModelGraphRunner, which serve the Llama-shaped family with padded batches.

Precision.  The residual stream, every norm, rotation, softmax, decay, gate of a recurrence and the
recurrent state are fp32.  Projections take their operand in the activation type (bf16, or fp32 when
the runner is built with dtype=float32 - then nothing at all is rounded to 16 bits) and leave fp32
accumulators; cached keys and values are of the activation type.

Per layer (Pagazen):
  mamba2    in-projection -> conv+SiLU over x|B|C (tail kept per slot) -> softplus step / decay ->
            outer-product scan (state per slot) -> SiLU(z) gate, grouped unit-RMS, weight -> out-projection
  parallel  left: fused q|k|v projection -> unit-RMS of q and k per head, k/v into the pages ->
            windowed softmax attention with distance penalty -> out-projection
            right: fused q|k|v|g projection -> rotate q,k (k scaled) -> fixed-decay scan ->
            unit-RMS per head, SiLU(g) gate -> out-projection
  then      x += unit_rms(sublayer output) * (1 + w)  (both mixers of a parallel layer enter one norm)
  mlp       up -> relu^2 -> down -> the same post-norm residual step
"""
import logging
from typing import Dict, List, Optional

import torch

from ...kernel import ragged_ops as ops
from ...models.pagazen import PagazenConfig, mamba2_sizes
from ..state_cache import HybridCacheManager, RaggedStep

logger = logging.getLogger(__name__)


class RaggedRunner:
    PAGE = 64

    def __init__(self, model, device="cuda", dtype=torch.bfloat16, wave_tiles: bool = True,
                 chunked_scan: bool = True, graphs: bool = True, max_graph_rows: int = 64, tiled_attn: bool = True):
        """`wave_tiles` / `chunked_scan` = False keep every projection on the plain any-shape kernel and
        every recurrence token by token, `tiled_attn` = False every token on the plain attention kernel (the
        forms the faster ones are checked against).  `graphs`:
        steps in which every row brings one token (decoding) are captured once per row count into a
        hipGraph and replayed - some seventy launches become one."""
        assert dtype in (torch.bfloat16, torch.float32)
        self.chunked_scan, self.tiled_attn = chunked_scan, tiled_attn
        self.use_graphs, self.max_graph_rows = graphs, max_graph_rows
        self._graphs: Dict[int, tuple] = {}
        self._arena, self._arena_off, self._measured = None, 0, 0
        self.model, self.cfg, self.device, self.dtype = model, model.config, device, dtype
        self.wave_tiles = wave_tiles
        cfg: PagazenConfig = self.cfg
        self.vocab_size, self.width = cfg.vocab_size, cfg.width
        self.weight_bytes = 0
        self._w: Dict[int, dict] = {}
        for i, layer in enumerate(cfg.layers):
            if cfg.weights_layer(i) == i:
                self._w[i] = self._prepare_layer(i, layer)
        self.embed = self._act(model.get("embed"))
        self.final_norm = self._small(model.get("final.norm"))
        self.head = self._linear(model.get("head"))

    # ------------------------------------------------------------------ weights
    def _act(self, t):
        return t.to(device=self.device, dtype=self.dtype).contiguous()

    def _small(self, t):
        return t.to(device=self.device, dtype=torch.float32).contiguous()

    def _linear(self, *parts):
        w = torch.cat([self._act(p) for p in parts], dim=0) if len(parts) > 1 else self._act(parts[0])
        lin = ops.AnyLinear(w, wave_tiles=self.wave_tiles)
        self.weight_bytes += lin.nbytes
        return lin

    def _prepare_layer(self, i: int, layer: dict) -> dict:
        g, p, m = self.model.get, f"l{i}.", layer["mixer"]
        w = {"norm1": self._small(g(p + "norm1"))}
        if layer["type"] == "mamba2":
            w.update(sizes=mamba2_sizes(m), w_in=self._linear(g(p + "mix.in")), conv=self._small(g(p + "mix.conv")),
                     conv_b=self._small(g(p + "mix.conv.b")), dt_bias=self._small(g(p + "mix.dt_bias")),
                     a_log=self._small(g(p + "mix.A_log")), skip=self._small(g(p + "mix.D")),
                     norm=self._small(g(p + "mix.norm")), w_o=self._linear(g(p + "mix.o")))
        else:
            L, R = m["left"], m["right"]
            H = int(L["heads"])
            slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float64)
            rot = int(R["rot"]["dims"])
            inv_freq = float(R["rot"]["base"]) ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)
            w.update(left_qkv=self._linear(g(p + "mix.left.q"), g(p + "mix.left.k"), g(p + "mix.left.v")),
                     left_o=self._linear(g(p + "mix.left.o")), slopes=self._small(slopes),
                     right_qkvg=self._linear(g(p + "mix.right.q"), g(p + "mix.right.k"), g(p + "mix.right.v"),
                                             g(p + "mix.right.g")),
                     right_o=self._linear(g(p + "mix.right.o")),
                     decay=self._small(torch.tensor([float(x) for x in R["decay"]], dtype=torch.float64)),
                     log_decay=self._small(torch.log(torch.tensor([float(x) for x in R["decay"]], dtype=torch.float64))),
                     inv_freq=inv_freq.to(self.device))
            assert len(R["decay"]) == int(R["heads"]), "one decay per retention head"
        if layer.get("mlp"):
            w.update(norm2=self._small(g(p + "norm2")), up=self._linear(g(p + "mlp.up")),
                     down=self._linear(g(p + "mlp.down")))
        return w

    # ------------------------------------------------------------------ cache geometry
    def cache_layout(self):
        """(kv_layers, state_layers) for HybridCacheManager: what every layer RUN keeps per sequence."""
        kv, state = {}, {}
        for i, layer in enumerate(self.cfg.layers):
            m = layer["mixer"]
            if layer["type"] == "mamba2":
                s = mamba2_sizes(m)
                state[i] = {"conv": (max(s["taps"] - 1, 0), s["conv_ch"]), "ssm": (s["heads"], s["n"], s["p"])}
            else:
                L, R = m["left"], m["right"]
                kv[i] = (int(L["kv_heads"]), int(L["dim"]), int(L["vdim"]))
                state[i] = {"ret": (int(R["heads"]), int(R["dim"]), int(R["vdim"]))}
        return kv, state

    def make_cache(self, n_pages: int, n_slots: int, max_tokens: int = 4096, max_rows: int = 32,
                   max_step_tokens: int = 8192) -> HybridCacheManager:
        kv, state = self.cache_layout()
        return HybridCacheManager(n_pages, self.PAGE, n_slots, kv, state, dtype=self.dtype, device=self.device,
                                  max_tokens=max_tokens, max_rows=max_rows, max_step_tokens=max_step_tokens)

    # ------------------------------------------------------------------ layers
    def _take(self, rows, cols, dtype):
        """A [rows, cols] buffer: from the arena of the step being captured or replayed (the same
        addresses every time), else a fresh allocation."""
        nbytes = (rows * cols * (4 if dtype == torch.float32 else 2) + 255) // 256 * 256
        self._measured += nbytes
        if self._arena is None:
            return torch.empty(rows, cols, dtype=dtype, device=self.device)
        assert self._arena_off + nbytes <= self._arena.numel(), "step arena too small"
        t = self._arena[self._arena_off:self._arena_off + nbytes].view(dtype)[:rows * cols].view(rows, cols)
        self._arena_off += nbytes
        return t

    def _f32buf(self, rows, cols):
        return self._take(rows, cols, torch.float32)

    def _actbuf(self, rows, cols):
        return self._take(rows, cols, self.dtype)

    def _mamba2(self, li, w, h, step: RaggedStep, cache: HybridCacheManager):
        s, T, eps = w["sizes"], step.tokens, self.cfg.eps
        inner, ch, H, N, P, G = s["inner"], s["conv_ch"], s["heads"], s["n"], s["p"], s["groups"]
        st = cache.states[li]
        proj = w["w_in"](h, self._f32buf(T, w["w_in"].n))     # [z | x B C | dt]
        xbc = self._f32buf(T, ch)
        ops.conv_silu(proj[:, inner:inner + ch], st["conv"], w["conv"], w["conv_b"], xbc, step)
        gain, decay, log_decay = self._f32buf(T, H), self._f32buf(T, H), self._f32buf(T, H)
        ops.softplus_decay(proj[:, inner + ch:inner + ch + H], w["dt_bias"], w["a_log"], gain, decay, log_decay)
        y = self._f32buf(T, inner)
        ops.scan_outer(q=xbc[:, inner + G * N:], k=xbc[:, inner:inner + G * N], v=xbc[:, :inner], decay=decay,
                       gain=gain, skip=w["skip"], state=st["ssm"], out=y, step=step, heads=H, n=N, p=P,
                       q_div=H // G, k_div=H // G, log_decay=log_decay, chunked=self.chunked_scan)
        u = self._actbuf(T, inner)
        ops.gated_group_norm(y, proj[:, :inner], w["norm"], u, groups=s["norm_groups"], gate_first=True, eps=eps)
        return w["w_o"](u, self._f32buf(T, self.width)), None

    def _parallel(self, li, w, m, h, step: RaggedStep, cache: HybridCacheManager):
        T, eps = step.tokens, self.cfg.eps
        L, R = m["left"], m["right"]
        H, G, d, dv = int(L["heads"]), int(L["kv_heads"]), int(L["dim"]), int(L["vdim"])
        qkv = w["left_qkv"](h, self._f32buf(T, w["left_qkv"].n))
        kc, vc = cache.k_caches[li], cache.v_caches[li]
        ops.qk_unitnorm_store(qkv, kc, vc, step, H, G, d, dv, eps)
        a = self._actbuf(T, H * dv)
        ops.window_attn(qkv, kc, vc, a, step, w["slopes"], H, G, d, dv, float(L["scale"]), int(L["mask"]["size"]),
                        tiled=self.tiled_attn)
        left = w["left_o"](a, self._f32buf(T, self.width))

        Hr, dr, dvr, rot = int(R["heads"]), int(R["dim"]), int(R["vdim"]), int(R["rot"]["dims"])
        qkvg = w["right_qkvg"](h, self._f32buf(T, w["right_qkvg"].n))
        q, k = qkvg[:, :Hr * dr], qkvg[:, Hr * dr:2 * Hr * dr]
        v, g = qkvg[:, 2 * Hr * dr:2 * Hr * dr + Hr * dvr], qkvg[:, 2 * Hr * dr + Hr * dvr:]
        ops.rotary_pairs_(q, w["inv_freq"], step.tok_pos, Hr, dr, rot, 1.0)
        ops.rotary_pairs_(k, w["inv_freq"], step.tok_pos, Hr, dr, rot, dr ** -0.5)
        o = self._f32buf(T, Hr * dvr)
        ops.scan_outer(q=q, k=k, v=v, decay=w["decay"], gain=None, skip=None, state=cache.states[li]["ret"], out=o,
                       step=step, heads=Hr, n=dr, p=dvr, log_decay=w["log_decay"], chunked=self.chunked_scan)
        u = self._actbuf(T, Hr * dvr)
        ops.gated_group_norm(o, g, None, u, groups=Hr, gate_first=False, eps=eps)
        return left, w["right_o"](u, self._f32buf(T, self.width))

    @torch.inference_mode()
    def forward(self, step: RaggedStep, cache: HybridCacheManager, want: Optional[torch.Tensor] = None,
                residuals: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
        """Run the step; returns fp32 logits [len(want), vocab] for the token indices in `want` (int32 on
        the device; None = every token).  `residuals` receives a copy of the stream after every layer
        run (debugging and tests)."""
        if (self.use_graphs and residuals is None and step.tokens == step.rows <= self.max_graph_rows):
            return self._replay(step, cache, want)
        return self._run(step, cache, want, residuals)

    # ------------------------------------------------------------------ captured decoding steps
    def _replay(self, step: RaggedStep, cache: HybridCacheManager, want):
        B = step.rows
        key = (B, id(cache))
        if key not in self._graphs:
            try:
                self._graphs[key] = self._capture(step, cache)
            except Exception as e:   # the recording failed (nothing of it ran): this row count stays uncaptured
                logger.warning("decoding steps of %d rows are not captured: %r", B, e)
                self._graphs[key] = None
        entry = self._graphs[key]
        if entry is None:
            return self._run(step, cache, want, None)
        graph, logits = entry[0], entry[2]
        graph.replay()
        if want is None:
            return logits.clone()
        return logits.index_select(0, want.long())

    def _capture(self, step: RaggedStep, cache: HybridCacheManager):
        """One run of the step on a side stream with fresh allocations (it sizes the arena and lets the
        projections set up their per-stream workspaces), the recurrent state of the step's slots put back
        as it was, then the same launches recorded over an arena.  Everything a replay reads that
        changes from step to step - tokens, positions, slots, block table - lies in the cache manager's
        one device buffer; keys and values of the step are written again by the replay with the same
        contents."""
        import ctypes
        from ... import _native as nv
        from .model_graph import HipGraph
        B, slots = step.rows, list(step.slots)
        idx = torch.tensor(slots, dtype=torch.long, device=self.device)
        saved = [(t, t.index_select(0, idx)) for named in cache.states.values() for t in named.values()]
        all_rows = torch.arange(B, dtype=torch.int32, device=self.device)
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._arena, self._measured = None, 0
            try:
                self._run(step, cache, all_rows, None)
            finally:   # whatever that run did to the slots' state is undone: the step itself is still to come
                for t, old in saved:
                    t.index_copy_(0, idx, old)
            arena = torch.empty(self._measured + 4096, dtype=torch.uint8, device=self.device)
            side.synchronize()
            self._arena, self._arena_off = arena, 0
            nv.check("mv_graph_begin_capture", nv.lib().mv_graph_begin_capture(side.cuda_stream))
            try:
                logits = self._run(step, cache, all_rows, None)
            finally:
                handle = ctypes.c_void_p()
                rc = nv.lib().mv_graph_end_capture(side.cuda_stream, ctypes.byref(handle))
                self._arena = None
            nv.check("mv_graph_end_capture", rc)
        torch.cuda.current_stream().wait_stream(side)
        logger.info("captured a decoding step of %d rows (%d KiB of intermediates)", B, arena.numel() >> 10)
        return HipGraph(handle), arena, logits, all_rows      # the arena and the row list stay alive with the graph

    def _run(self, step: RaggedStep, cache: HybridCacheManager, want, residuals) -> torch.Tensor:
        cfg, T = self.cfg, step.tokens
        x, h = self._f32buf(T, self.width), self._actbuf(T, self.width)
        ops.embed_scaled(self.embed, step.ids, cfg.embed_scale, x, h)
        for li, layer in enumerate(cfg.layers):
            w, m = self._w[cfg.weights_layer(li)], layer["mixer"]
            if layer["type"] == "mamba2":
                y1, y2 = self._mamba2(li, w, h, step, cache)
                ops.postnorm_residual(y1, w["norm1"], cfg.eps, x, h)
            else:
                y1, y2 = self._parallel(li, w, m, h, step, cache)
                ops.postnorm_residual(y1, w["norm1"], cfg.eps, x, h, y2=y2, s1=float(m["left_scale"]),
                                      s2=float(m["right_scale"]))
            if layer.get("mlp"):
                up = w["up"](h, self._f32buf(T, w["up"].n))
                act = self._actbuf(T, up.shape[1])
                ops.relu_squared(up, act)
                ops.postnorm_residual(w["down"](act, self._f32buf(T, self.width)), w["norm2"], cfg.eps, x, h)
            if residuals is not None:
                residuals.append(x.clone())
        rows = T if want is None else want.numel()
        normed = self._actbuf(rows, self.width)
        if rows == 0:
            return self._f32buf(0, self.vocab_size)
        ops.offset_rmsnorm_gather(x, want, self.final_norm, cfg.eps, normed)
        logits = self.head(normed, self._f32buf(rows, self.vocab_size))
        if cfg.logit_softcap:
            ops.softcap_(logits, cfg.logit_softcap)
        return logits
