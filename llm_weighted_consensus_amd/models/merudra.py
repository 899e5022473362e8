"""Merudra decoder on the fp32-residual kernel set (``ops/res32.py``, ``csrc/kernels/res32``).

The residual stream x is fp32.  A layer (T rows of a step: decode rows and prompt-portion rows alike):

    h1, xb = x + conv_t(x), cast(x)                  res32.conv_hist (per-sequence history slot)
    r1     = xb @ Wrg1^T + b                          gate logits of the mixer's result
    proj   = h1 @ [Wq | Wk | Wg]^T (+ biases)         ONE GEMM       (delta: [Wq | Wk | Wv | Wb | Wa | Wg])
    attention layer:
      q    = per-head unit-RMS q * scale * temp(p);   res32.head_norm_kv_write (normalised k -> paged K cache,
                                                      k as projected -> paged V cache: the values are the keys)
      a    = causal softmax attention over the cache  res32.window_attn (no distance bias, unbounded window)
      a   *= sigmoid(proj_g)                          res32.gate_mul
    delta layer:
      qkv  = silu(conv_t([q | k | v]))                res32.conv_hist (short convolution, history slot), fp32
      o    = gated delta rule over the state slot     res32.delta_rule (state fp32 [H, D, Dv] per sequence)
      a    = o / rms(o) * w * silu(proj_g)            res32.head_norm_gate
    x     += rms_norm(sigmoid(r1) * (a @ Wo^T)) * w1  res32.gated_norm_residual
    h2, xb = x + conv_t(x), cast(x)                   res32.conv_hist
    route  = softmax(h2 @ Wr^T) (+ correction), top-k res32.router (fp32; identity experts beyond the real ones)
    y      = sum_j s_j expert_j(h2)                   res32.expert_rows / the grouped MFMA GEMMs, res32.moe_combine
    x     += rms_norm(sigmoid(r2) * y) * w2           res32.gated_norm_residual
    x     += rms_norm(Wp (gelu(Ws x) * e_l[token]))*w res32.gelu_mul_rows, res32.gated_norm_residual (no gate)
    X[l+1] = x;  next x = sum_j c_l[j] X[j]           res32.stack_mix (all layer results stay resident)

Per-sequence state besides the K/V pages (the convolutions' last inputs and the delta layers' matrices) lives in a
:class:`..models.state.RecurrentStatePool`; the engine's block manager hands out its slots.

``dtype=torch.float32`` runs every GEMM, activation and the cache in true fp32; bf16 is the serving mode.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable, Dict, List, Optional

import numpy as np
import torch
import torch.nn.functional as F

from .. import ops
from ..ops import gemm_plan, res32
from .cache import PagedLayerCache
from .config import MerudraConfig
from .state import RecurrentStatePool

UNBOUNDED = 1 << 30  # "window" of a causal attention without one


@dataclass
class MerudraLayer:
    canon1: torch.Tensor                 # fp32 [d, taps]
    canon2: Optional[torch.Tensor]
    w_rg1: torch.Tensor
    b_rg1: torch.Tensor
    w_rg2: Optional[torch.Tensor]
    b_rg2: Optional[torch.Tensor]
    w_in: torch.Tensor                   # fused input-side projections of the mixer
    b_in: Optional[torch.Tensor]
    w_o: torch.Tensor
    norm1: torch.Tensor                  # fp32
    norm2: Optional[torch.Tensor]
    side_gate: torch.Tensor
    side_proj: torch.Tensor
    side_norm: torch.Tensor              # fp32
    dwa: torch.Tensor                    # fp32 [l + 2]
    extra: Dict[str, torch.Tensor] = field(default_factory=dict)   # delta: conv, A_log, dt_bias, norm; moe: router, ...


class MerudraModel:
    paged_prefill = True      # whole prompts run as one portion over the paged cache (engine._run_prefill)
    supports_cascade = False
    graph_safe = True
    float_logits = True
    has_state = True          # the engine gives every sequence a recurrent-state slot

    # experts at least this large (d * ff) go through the grouped matrix-core GEMMs of the full kernel extension;
    # smaller ones are read whole from cache by the row kernel faster than a 128-row tile is filled
    GROUPED_MIN = 1 << 18

    def __init__(self, cfg: MerudraConfig, device="cuda", dtype=torch.bfloat16, seed: int = 0,
                 weights_path: Optional[str] = None, max_position: Optional[int] = None):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Merudra runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        if self.device.type != "cuda":
            raise RuntimeError("Merudra runs on the GPU kernels only (no CPU path)")
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        if cfg.canon_taps < 1 or cfg.canon_taps > 16:
            raise ValueError("Merudra: canon.taps must be in 1..16")
        for L in cfg.layer_specs:
            if L.type == "delta" and (L.mixer.dim > res32.kernels().delta_rule_max_dim() or not 1 <= L.mixer.conv <= 16):
                raise ValueError("Merudra: delta layer sizes beyond what the kernels are built for")
            if L.mlp is not None and L.mlp.experts + L.mlp.identity > res32.kernels().router_max_outputs():
                raise ValueError("Merudra: too many router outputs")
        self.logit_width = -(-cfg.vocab_size // 32) * 32
        self.cache_index = {li: ci for ci, li in enumerate(cfg.attention_layers)}
        self._mm32 = self._probe_mm32()
        raw = self._read(weights_path) if weights_path else self._random(seed)
        self._assemble(raw)
        self.g8_ws = None
        self.on_layer: Optional[Callable[[int, torch.Tensor], None]] = None
        self._zeros_h: Dict[int, torch.Tensor] = {}

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self) -> dict:
        """name -> shape of every tensor of a checkpoint of this config."""
        cfg, d = self.cfg, self.cfg.hidden
        out = {"embed": (cfg.vocab_size, d), "side.embed": (cfg.vocab_size, cfg.side_dim * cfg.layers), "final.norm": (d,),
               "head": (cfg.vocab_size, d)}
        for i, L in enumerate(cfg.layer_specs):
            m, p = L.mixer, f"l{i}."
            out.update({p + "norm1": (d,), p + "canon1": (d, cfg.canon_taps), p + "rg1": (d, d), p + "rg1.b": (d,),
                        p + "dwa": (i + 2,), p + "side.gate": (cfg.side_dim, d), p + "side.proj": (d, cfg.side_dim),
                        p + "side.norm": (d,)})
            if L.type == "attention":
                out.update({p + "mix.q": (m.nq, d), p + "mix.q.b": (m.nq,), p + "mix.k": (m.nk, d), p + "mix.k.b": (m.nk,),
                            p + "mix.g": (m.heads * m.vdim, d), p + "mix.o": (d, m.heads * m.vdim)})
            else:
                out.update({p + "mix.q": (m.nq, d), p + "mix.q.conv": (m.nq, m.conv), p + "mix.k": (m.nq, d),
                            p + "mix.k.conv": (m.nq, m.conv), p + "mix.v": (m.nv, d), p + "mix.v.conv": (m.nv, m.conv),
                            p + "mix.b": (m.heads, d), p + "mix.a": (m.heads, d), p + "mix.A_log": (m.heads,),
                            p + "mix.dt_bias": (m.heads,), p + "mix.norm": (m.vdim,), p + "mix.g": (m.nv, d),
                            p + "mix.o": (d, m.nv)})
            if L.mlp is not None:
                e = L.mlp
                out.update({p + "norm2": (d,), p + "canon2": (d, cfg.canon_taps), p + "rg2": (d, d), p + "rg2.b": (d,),
                            p + "mlp.router": (e.experts + e.identity, d), p + "mlp.correction": (e.experts + e.identity,)})
                for x in range(e.experts):
                    out.update({f"{p}mlp.e{x}.gate": (e.ff, d), f"{p}mlp.e{x}.up": (e.ff, d), f"{p}mlp.e{x}.down": (d, e.ff)})
        return out

    def _random(self, seed: int) -> dict:
        """Random weights of the config's shapes (benchmarks, tests): bf16-representable values."""
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        d = self.cfg.hidden
        out = {}
        for name, shape in self.tensor_shapes().items():
            leaf = name.split(".")[-1]
            if leaf in ("norm1", "norm2", "norm") or name == "final.norm":
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            elif leaf in ("canon1", "canon2"):
                t = 0.2 * torch.randn(shape, generator=g)
            elif leaf == "conv":
                t = 0.5 * torch.randn(shape, generator=g)
            elif leaf == "b" and len(shape) == 1:
                t = 0.1 * torch.randn(shape, generator=g)
            elif leaf == "dwa":
                t = 0.15 * torch.randn(shape, generator=g)
                t[-1] += 1.0
            elif leaf == "A_log":
                t = torch.rand(shape, generator=g) * 2 - 1
            elif leaf == "dt_bias":
                t = torch.randn(shape, generator=g)
            elif leaf == "correction":
                t = 0.05 * torch.randn(shape, generator=g)
            elif name in ("embed", "side.embed"):
                t = torch.randn(shape, generator=g)
            else:
                t = torch.randn(shape, generator=g) / math.sqrt(shape[-1] if len(shape) > 1 else d)
            out[name] = t.to(torch.bfloat16)
        return out

    def _read(self, path: str) -> dict:
        from safetensors.torch import load_file

        p = Path(path)
        files = sorted(p.glob("*.safetensors")) if p.is_dir() else [p]
        if not files:
            raise FileNotFoundError(f"no .safetensors under {path}")
        sd = {}
        for f in files:
            sd.update(load_file(str(f), device="cpu"))
        for name, shape in self.tensor_shapes().items():
            if name not in sd:
                raise KeyError(f"{path}: tensor {name} missing")
            if tuple(sd[name].shape) != tuple(shape):
                raise ValueError(f"{path}: {name} has shape {tuple(sd[name].shape)}, the config says {tuple(shape)}")
        return sd

    def _assemble(self, sd: dict) -> None:
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def t(name):
            return sd[name].to(device=dev, dtype=dt).contiguous()

        def f32(name):
            return sd[name].to(device=dev, dtype=torch.float32).contiguous()

        def taps_major(w):
            """[C, taps] convolution weights stored tap-major (the kernels' 16-byte path reads w[j][c : c + 4])."""
            return w.t().contiguous().t()

        self.embed, self.side_embed = t("embed"), t("side.embed")
        self.final_w, self.head = f32("final.norm"), t("head")
        self.layers: List[MerudraLayer] = []
        for i, L in enumerate(cfg.layer_specs):
            m, p = L.mixer, f"l{i}."
            extra: Dict[str, torch.Tensor] = {}
            if L.type == "attention":
                w_in = torch.cat([t(p + "mix.q"), t(p + "mix.k"), t(p + "mix.g")], 0).contiguous()
                b_in = torch.cat([t(p + "mix.q.b"), t(p + "mix.k.b"), torch.zeros(m.heads * m.vdim, dtype=dt, device=dev)])
            else:
                w_in = torch.cat([t(p + "mix.q"), t(p + "mix.k"), t(p + "mix.v"), t(p + "mix.b"), t(p + "mix.a"),
                                  t(p + "mix.g")], 0).contiguous()
                b_in = None
                extra["conv"] = taps_major(torch.cat([f32(p + "mix.q.conv"), f32(p + "mix.k.conv"), f32(p + "mix.v.conv")], 0))
                extra["A_log"], extra["dt_bias"], extra["norm"] = f32(p + "mix.A_log"), f32(p + "mix.dt_bias"), f32(p + "mix.norm")
            if L.mlp is not None:
                e = L.mlp
                extra["router"], extra["correction"] = f32(p + "mlp.router"), f32(p + "mlp.correction")
                if self._mm32 and bool((extra["router"].to(dt).float() == extra["router"]).all()):
                    extra["router_t"] = extra["router"].to(dt).t().contiguous()
                else:
                    self._mm32 = False
                if e.experts:
                    extra["w_gu"] = torch.stack([torch.cat([t(f"{p}mlp.e{x}.gate"), t(f"{p}mlp.e{x}.up")], 0)
                                                 for x in range(e.experts)]).contiguous()
                    extra["w_down"] = torch.stack([t(f"{p}mlp.e{x}.down") for x in range(e.experts)]).contiguous()
                else:
                    extra["w_gu"] = torch.zeros(0, 2 * e.ff, cfg.hidden, dtype=dt, device=dev)
                    extra["w_down"] = torch.zeros(0, cfg.hidden, e.ff, dtype=dt, device=dev)
            has = L.mlp is not None
            self.layers.append(MerudraLayer(
                canon1=taps_major(f32(p + "canon1")), canon2=taps_major(f32(p + "canon2")) if has else None, w_rg1=t(p + "rg1"), b_rg1=t(p + "rg1.b"),
                w_rg2=t(p + "rg2") if has else None, b_rg2=t(p + "rg2.b") if has else None, w_in=w_in, b_in=b_in,
                w_o=t(p + "mix.o"), norm1=f32(p + "norm1"), norm2=f32(p + "norm2") if has else None,
                side_gate=t(p + "side.gate"), side_proj=t(p + "side.proj"), side_norm=f32(p + "side.norm"),
                dwa=f32(p + "dwa"), extra=extra))

    # ------------------------------------------------------------------ GEMMs
    def _probe_mm32(self) -> bool:
        """Whether this torch build multiplies bf16 matrices into an fp32 result (the router's logits)."""
        if self.dtype != torch.bfloat16:
            return False
        try:
            a = torch.zeros(8, 16, dtype=self.dtype, device=self.device)
            return torch.mm(a, a.t(), out_dtype=torch.float32).dtype == torch.float32
        except (TypeError, RuntimeError):
            return False

    def _linear(self, x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
        if b is None and self.g8_ws is not None:
            return gemm_plan.linear(x, w, ws=self.g8_ws)
        return F.linear(x, w, b)

    def tune_gemms(self, M: int, bucket: bool = False, lm_head: bool = True, only=None) -> None:
        """Pick the backend of the bias-free projections at M rows by timing the library and the hand-written
        cores (the engine calls this before it captures a decode bucket's graph).  bf16 only, and only where the
        full kernel extension is built; otherwise every GEMM stays on the library."""
        if self.dtype != torch.bfloat16 or only is not None or not ops.available():
            return
        if self.g8_ws is None:
            self.g8_ws = ops.new_gemm8p_workspace(self.device)
        seen = set()
        for L in self.layers:
            for w in (L.w_o, L.side_gate, L.side_proj) + ((L.w_in,) if L.b_in is None else ()):
                if tuple(w.shape) not in seen and w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0:
                    seen.add(tuple(w.shape))
                    gemm_plan.tune(torch.randn(M, w.shape[1], device=self.device).to(self.dtype), w, ws=self.g8_ws, bucket=bucket)
        if lm_head:
            gemm_plan.tune(torch.randn(M, self.cfg.hidden, device=self.device).to(self.dtype), self.head, ws=self.g8_ws,
                           bucket=bucket)

    # ------------------------------------------------------------------ cache and state
    def _layer_dims(self):
        return [(self.cfg.layer_specs[li].mixer.nk, self.cfg.layer_specs[li].mixer.nv) for li in self.cfg.attention_layers]

    def new_cache(self, num_blocks: int, block_size: int) -> PagedLayerCache:
        return PagedLayerCache(self._layer_dims(), num_blocks, block_size, self.device, self.dtype)

    def bytes_per_block(self, block_size: int) -> int:
        n = PagedLayerCache.elems_per_block(self._layer_dims(), block_size) * (4 if self.dtype == torch.float32 else 2)
        return max(n, 16)

    def state_fields(self):
        """(name, shape) of every per-sequence state tensor: the input convolutions' last inputs per sublayer, the
        delta layers' short-convolution inputs and their matrices."""
        cfg, d, k = self.cfg, self.cfg.hidden, self.cfg.canon_taps - 1
        out = []
        for i, L in enumerate(cfg.layer_specs):
            out.append((f"c1.{i}", (k, d)))
            if L.mlp is not None:
                out.append((f"c2.{i}", (k, d)))
            if L.type == "delta":
                m = L.mixer
                out.append((f"dc.{i}", (m.conv - 1, 2 * m.nq + m.nv)))
                out.append((f"S.{i}", (m.heads, m.dim, m.vdim)))
        return out

    def new_state(self, num_slots: int) -> RecurrentStatePool:
        return RecurrentStatePool(self.state_fields(), num_slots, self.device)

    def bytes_per_state_slot(self) -> int:
        return RecurrentStatePool.bytes_per_slot(self.state_fields())

    # ------------------------------------------------------------------ forward
    def _experts(self, h2: torch.Tensor, L: MerudraLayer, e) -> torch.Tensor:
        """Routed experts of the rows h2 -> fp32 [T, d]."""
        x = L.extra
        if self._mm32:  # bf16 operands, fp32 accumulation AND output: the checkpoint's router is bf16-exact
            z = torch.mm(h2, x["router_t"], out_dtype=torch.float32)
        else:
            z = F.linear(h2.float(), x["router"])  # router logits in fp32
        _ids, w, row_off, src, row_expert, inv = res32.router(z, x["correction"], e.experts, e.top)
        d = self.cfg.hidden
        if (self.dtype == torch.bfloat16 and e.experts and d * e.ff >= self.GROUPED_MIN and d % 64 == 0 and e.ff % 64 == 0
                and ops.available()):
            rows = src.numel()
            gu = ops.grouped_gemm(h2, x["w_gu"], row_off, a_rows=src, rows=rows)
            Y = ops.grouped_gemm(ops.silu_mul(gu), x["w_down"], row_off)
        else:
            Y = res32.expert_rows(h2, src, row_expert, row_off, x["w_gu"], x["w_down"])
        return res32.moe_combine(Y, inv, w, h2)

    def _forward(self, tokens, positions, slots, cache: PagedLayerCache, state: RecurrentStatePool,
                 items: res32.StepItems, attend, keep: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Every layer over the step's rows; ``attend(q, li, out)`` runs the attention of layer ``li`` into ``out``.
        Returns the fp32 stream that the output norm reads, [T, d].

        ``keep`` (int64 rows): only these rows' final states are wanted (a prompt's last token).  The LAST layer
        then still runs its mixer and both input convolutions on every row (keys, values, the recurrent state and
        the convolutions' histories are what later steps read), but the gate, the routed experts, the token input
        and the layer mix on the kept rows only; returns [len(keep), d]."""
        cfg, dt = self.cfg, self.dtype
        T, d, eps, nl = tokens.shape[0], cfg.hidden, cfg.norm_eps, len(self.layers)
        exact = dt == torch.float32
        X = torch.empty(nl + 1, T, d, dtype=torch.float32, device=self.device)  # every layer's result stays resident
        res32.embed_rows(self.embed, tokens, X[0])
        X[1].copy_(X[0])
        xb = None if exact else torch.empty(T, d, dtype=dt, device=self.device)
        for li, (S, L) in enumerate(zip(cfg.layer_specs, self.layers)):
            m, x = S.mixer, X[li + 1]
            short = keep is not None and li + 1 == nl
            h = torch.empty(T, d, dtype=dt, device=self.device)
            res32.conv_hist(x, L.canon1, state[f"c1.{li}"], items, h, mode=0, out2=xb)
            r = self._linear(x if exact else xb, L.w_rg1, L.b_rg1)
            proj = self._linear(h, L.w_in, L.b_in)
            a = torch.empty(T, m.heads * m.vdim, dtype=dt, device=self.device)
            if S.type == "attention":
                ci = self.cache_index[li]
                q = res32.head_norm_kv_write(proj, m.nq, m.nq, positions, slots, cache.k[ci], cache.v[ci], m.heads,
                                             m.kv_heads, eps, m.scale, m.temp_coef, m.temp_every)
                attend(q, li, a)
                res32.gate_mul(a, proj[:, m.nq + m.nk:], "sigmoid")
            else:
                nqkv = 2 * m.nq + m.nv
                qkv = torch.empty(T, nqkv, dtype=torch.float32, device=self.device)
                res32.conv_hist(proj[:, :nqkv], L.extra["conv"], state[f"dc.{li}"], items, qkv, mode=1)
                o = res32.delta_rule(qkv, proj, nqkv, nqkv + m.heads, L.extra["A_log"], L.extra["dt_bias"], state[f"S.{li}"],
                                     items, m.heads, m.kv_heads)
                res32.head_norm_gate(o, a, m.heads, eps, w=L.extra["norm"], gate=proj[:, nqkv + 2 * m.heads:], mode="silu")
            res32.gated_norm_residual(x, self._linear(a, L.w_o), L.norm1, eps, gate_logits=r,
                                      x_cast=xb if S.mlp is None else None)
            if S.mlp is not None:
                res32.conv_hist(x, L.canon2, state[f"c2.{li}"], items, h, mode=0, out2=xb)
            toks = tokens
            if short:  # from here on only the kept rows
                x, h, toks = x.index_select(0, keep), h.index_select(0, keep), tokens.index_select(0, keep)
                xb = None if exact else xb.index_select(0, keep)
            if S.mlp is not None:
                r = self._linear(x if exact else xb, L.w_rg2, L.b_rg2)
                res32.gated_norm_residual(x, self._experts(h, L, S.mlp), L.norm2, eps, gate_logits=r, x_cast=xb)
            g = res32.gelu_mul_rows(self._linear(x if exact else xb, L.side_gate), self.side_embed, li * cfg.side_dim, toks)
            res32.gated_norm_residual(x, self._linear(g, L.side_proj), L.side_norm, eps)
            if short:
                Xk = torch.cat([X[:nl].index_select(1, keep), x[None]], 0)
                final = torch.empty(keep.numel(), d, dtype=torch.float32, device=self.device)
                return res32.stack_mix(Xk, L.dwa, nl + 1, final)
            nxt = X[li + 2] if li + 1 < nl else torch.empty(T, d, dtype=torch.float32, device=self.device)
            res32.stack_mix(X, L.dwa, li + 2, nxt)
            if self.on_layer is not None:
                self.on_layer(li, nxt)
        return nxt

    def _logits(self, x: torch.Tensor, rows: Optional[torch.Tensor], float_logits: bool) -> torch.Tensor:
        h = res32.rmsnorm_rows(x, self.final_w, self.cfg.norm_eps, self.dtype, rows=rows)
        lg = self._linear(h, self.head).float()
        if float_logits:
            return lg
        V, Vp = self.cfg.vocab_size, self.logit_width
        if Vp == V:
            return lg.to(torch.bfloat16)
        out = torch.full((lg.shape[0], Vp), float("-inf"), dtype=torch.bfloat16, device=lg.device)
        out[:, :V] = lg
        return out

    def _no_bias(self, H: int) -> torch.Tensor:
        z = self._zeros_h.get(H)
        if z is None:
            z = self._zeros_h[H] = torch.zeros(H, dtype=torch.float32, device=self.device)
        return z

    def _attend(self, cache, positions, tables, cu_q=None, k_lens=None, max_q=0):
        def run(q, li, out, rows=slice(None)):
            m = self.cfg.layer_specs[li].mixer
            ci = self.cache_index[li]
            z = self._no_bias(m.heads)
            res32.window_attn(q[rows], cache.k[ci], cache.v[ci], positions[rows], tables, z, z, UNBOUNDED, out[rows],
                              m.heads, m.kv_heads, cu_q=cu_q, k_lens=k_lens, max_q=max_q, bias=None, cores=True)
        return run

    def decode(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, block_tables: torch.Tensor,
               ctx_lens: torch.Tensor, cache: PagedLayerCache, num_splits: int = 1, cascade_tiles=None,
               float_logits: bool = False, state: Optional[RecurrentStatePool] = None,
               state_slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One decode step for B sequences -> logits [B, V]; device tensors only (hipGraph-capturable).  Row b
        reads table row b and the state slot ``state_slots[b]``; its key range ends at its own position."""
        if state is None or state_slots is None:
            raise RuntimeError("Merudra: a decode step needs the recurrent-state pool and the rows' slots")
        items = res32.StepItems.rows(state_slots, positions)
        x = self._forward(tokens, positions, slots, cache, state, items, self._attend(cache, positions, block_tables))
        return self._logits(x, None, float_logits)

    def forward_mixed(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, cache: PagedLayerCache,
                      n_dec: int, dec: Optional[dict], chunk: Optional[dict], logit_rows: torch.Tensor,
                      float_logits: bool = False, state: Optional[RecurrentStatePool] = None,
                      state_slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """ONE forward over [n_dec decode rows || prompt-portion rows]: every projection is one GEMM over both, the
        recurrent kernels walk decode rows and portions alike as items; the attention runs per part over the paged
        cache that this step's rows were just written to.  ``state_slots``: int32, the slot of every decode row,
        then of every portion.  Logits of ``logit_rows``."""
        if state is None or state_slots is None:
            raise RuntimeError("Merudra: a step needs the recurrent-state pool and the sequences' slots")
        T = tokens.shape[0]
        q_lens = list(chunk["lens"][0]) if T > n_dec else []
        cu = np.concatenate([np.arange(n_dec, dtype=np.int64), n_dec + np.concatenate([[0], np.cumsum(q_lens, dtype=np.int64)])])
        if cu[-1] != T or state_slots.numel() != n_dec + len(q_lens):
            raise ValueError("Merudra: rows, portions and state slots disagree")
        row_item = np.concatenate([np.arange(n_dec, dtype=np.int64), n_dec + np.repeat(np.arange(len(q_lens)), q_lens)])
        dev = self.device
        items = res32.StepItems(torch.from_numpy(row_item.astype(np.int32)).to(dev), torch.from_numpy(cu.astype(np.int32)).to(dev),
                                state_slots, positions)
        dec_run = self._attend(cache, positions, dec["block_tables"]) if n_dec else None
        chk_run = (self._attend(cache, positions, chunk["block_tables"], cu_q=chunk["cu_q"], k_lens=chunk.get("k_lens"),
                                max_q=int(chunk.get("max_q", 0))) if T > n_dec else None)

        def attend(q, li, out):
            if dec_run is not None:
                dec_run(q, li, out, slice(0, n_dec))
            if chk_run is not None:
                chk_run(q, li, out, slice(n_dec, T))

        # prompt portions of which few rows are wanted (a prompt's last token): the last layer's gate, experts and
        # token input on those rows only
        keep = logit_rows if n_dec == 0 and self.on_layer is None and 4 * logit_rows.numel() <= T else None
        x = self._forward(tokens, positions, slots, cache, state, items, attend, keep=keep)
        return self._logits(x, None if keep is not None else logit_rows, float_logits)

    def prefill(self, tokens, positions, slots, cu_seqlens, max_seqlen, last_idx, cache, ctx=None):
        raise RuntimeError("Merudra prefills through forward_mixed over the paged cache (paged_prefill)")
