"""Madipel decoder on the fp32-residual kernel set (``ops/res32.py``, ``csrc/kernels/res32``).

A layer is PARALLEL: one LayerNorm (weight and bias) feeds both sublayers, ``x += m * (mixer(h) + ff(h))``, and the
residual stream x stays fp32.  Per layer (T rows of a step: decode rows and prompt-portion rows alike):

    h     = layernorm(x)                                   res32.layernorm (fp32 statistics)
    proj  = h @ [Wq | Wk | Wv | Wup]^T                     ONE GEMM over the fused input-side weight
    q, kv = whole-projection RMS norms, per-head scale,    res32.proj_norm_kv_write (fp32; k, v into the paged
            value blending across layers, cache write       cache, q into an fp32 buffer)
    attn  = windowed attention with the log distance bias  res32.window_attn -> columns [0, H*Dv) of `cat`
    act   = xIELU(proj[:, up columns])                     res32.xielu       -> columns [H*Dv, H*Dv + ff) of `cat`
    y     = cat @ [Wo | Wdown]^T                           ONE GEMM: mixer and feed-forward outputs summed in
                                                           the accumulators
    x    += m * y                                          res32.residual_add_scaled (fp32)

Positions enter through the sinusoidal vector added to the embedding and through the attention's distance bias
(no rotation).  The output is LayerNorm -> head GEMM -> logits * logit_scale (fp32).

Value blending: the first layer whose config says ``v_mix`` publishes its values v0 (per token, this step's
rows); every later such layer caches ``(1 - lam) v + lam v0``.  v0 lives only inside one forward.

``dtype=torch.float32`` runs every GEMM, activation and the cache in true fp32 (exact mode); bf16 is the serving
mode.  GEMMs go through the per-shape planner of the other decoders (``ops/gemm_plan.py``): the vendor library
(torch -> hipBLASLt) for untuned shapes and for fp32, and for a decode bucket whichever of the library and the
hand-written cores was timed faster before the bucket's hipGraph is captured (:meth:`MadipelModel.tune_gemms`).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import gemm_plan, res32
from .cache import PagedLayerCache
from .config import MadipelConfig


@dataclass
class MadipelLayer:
    norm_w: torch.Tensor
    norm_b: torch.Tensor
    w_in: torch.Tensor        # [nq + nk + nv + ff, d]: q | k | v | up rows
    w_out: torch.Tensor       # [d, H*Dv + ff]: o | down columns
    q_norm: torch.Tensor      # [nq]
    k_norm: torch.Tensor      # [nk]
    head_scale: torch.Tensor  # fp32 [H]: softmax scale * the head's temperature
    r1: torch.Tensor          # fp32 [H]
    r2: torch.Tensor          # fp32 [H]
    vmix: torch.Tensor        # [1] blend weight (activation dtype)
    act: Optional[torch.Tensor]  # [2] xIELU parameters, None without a feed-forward
    vmode: int = 0            # 0 plain, 1 publishes v0, 2 blends with v0
    bias: Optional[torch.Tensor] = None  # fp32 [H, window] distance-bias table (matrix-core prompt kernel)


class MadipelModel:
    paged_prefill = True      # whole prompts run as one portion over the paged cache (engine._run_prefill)
    supports_cascade = False  # no shared-prefix cascade kernel for this attention
    graph_safe = True
    float_logits = True       # forward_mixed / decode return fp32 logits when asked (float_logits=True)

    def __init__(self, cfg: MadipelConfig, device="cuda", dtype=torch.bfloat16, seed: int = 0,
                 weights_path: Optional[str] = None, max_position: Optional[int] = None):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Madipel runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        if self.device.type != "cuda":
            raise RuntimeError("Madipel runs on the GPU kernels only (no CPU path)")
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False  # true fp32 products
        mixing = [L.mixer.nv for L in cfg.layer_specs if L.mixer.v_mix]
        if len(set(mixing)) > 1:
            raise ValueError("Madipel: layers that blend values must share kv_heads * vdim")
        # the sampler reads logits in words of 32 columns: other vocabularies get -inf columns up to the next 32
        self.logit_width = -(-cfg.vocab_size // 32) * 32
        self.inv_freq = res32.sinpos_inv_freq(cfg.hidden, cfg.sinpos_base, self.device)
        raw = self._read(weights_path) if weights_path else self._random(seed)
        self._assemble(raw)
        self.g8_ws = None  # the hand-written GEMM cores' workspace, made when a shape is first tuned
        self._split_ok = self._probe_split()
        # called with (layer index, residual stream) after every layer when set (bring-up, tests)
        self.on_layer: Optional[Callable[[int, torch.Tensor], None]] = None

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self) -> dict:
        """name -> shape of every tensor of a checkpoint of this config."""
        cfg, d = self.cfg, self.cfg.hidden
        out = {"embed": (cfg.vocab_size, d), "final.norm": (d,), "final.norm.b": (d,), "head": (cfg.vocab_size, d)}
        for i, L in enumerate(cfg.layer_specs):
            m, p = L.mixer, f"l{i}."
            out.update({p + "norm1": (d,), p + "norm1.b": (d,), p + "mix.q": (m.nq, d), p + "mix.k": (m.nk, d),
                        p + "mix.v": (m.nv, d), p + "mix.q.norm": (m.nq,), p + "mix.k.norm": (m.nk,),
                        p + "mix.vmix": (), p + "mix.r1": (m.heads,), p + "mix.r2": (m.heads,),
                        p + "mix.temp": (m.heads,), p + "mix.o": (d, m.heads * m.vdim)})
            if L.mlp_kind:
                out.update({p + "mlp.up": (L.ff, d), p + "mlp.down": (d, L.ff), p + "mlp.act": (2,)})
        return out

    def _random(self, seed: int) -> dict:
        """Random weights of the config's shapes (benchmarks, tests): bf16-representable values."""
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        d = self.cfg.hidden
        out = {}
        for name, shape in self.tensor_shapes().items():
            leaf = name.split(".")[-1]
            if name.endswith("norm1") or name.endswith("final.norm") or leaf == "norm":
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            elif leaf == "b":
                t = 0.05 * torch.randn(shape, generator=g)
            elif leaf == "vmix":
                t = torch.rand(shape, generator=g) * 0.5
            elif leaf in ("r1", "r2"):
                t = 0.2 + torch.rand(shape, generator=g)
            elif leaf == "temp":
                t = 0.75 + 0.5 * torch.rand(shape, generator=g)
            elif leaf == "act":
                t = torch.randn(shape, generator=g) * 0.5
            elif name == "embed":
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
        want = self.tensor_shapes()
        for name, shape in want.items():
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

        self.embed = t("embed")
        self.final_w, self.final_b, self.head = t("final.norm"), t("final.norm.b"), t("head")
        self.layers: List[MadipelLayer] = []
        published = False
        for i, L in enumerate(cfg.layer_specs):
            m, p = L.mixer, f"l{i}."
            rows = [t(p + "mix.q"), t(p + "mix.k"), t(p + "mix.v")]
            cols = [t(p + "mix.o")]
            if L.mlp_kind:
                rows.append(t(p + "mlp.up"))
                cols.append(t(p + "mlp.down"))
            vmode = 0
            if m.v_mix:
                vmode, published = (2 if published else 1), True
            self.layers.append(MadipelLayer(
                norm_w=t(p + "norm1"), norm_b=t(p + "norm1.b"), w_in=torch.cat(rows, 0).contiguous(),
                w_out=torch.cat(cols, 1).contiguous(), q_norm=t(p + "mix.q.norm"), k_norm=t(p + "mix.k.norm"),
                head_scale=(f32(p + "mix.temp") * m.scale).contiguous(), r1=f32(p + "mix.r1"), r2=f32(p + "mix.r2"),
                vmix=t(p + "mix.vmix").reshape(1), act=t(p + "mlp.act") if L.mlp_kind else None, vmode=vmode))
            Lw = self.layers[-1]
            if dt == torch.bfloat16 and m.heads * m.window <= (1 << 26) and res32.kernels().window_attn_mfma_ok(m.dim, m.vdim):
                Lw.bias = res32.distance_bias(Lw.r1, Lw.r2, m.window)

    # ------------------------------------------------------------------ GEMMs
    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        if self.g8_ws is not None:
            return gemm_plan.linear(x, w, ws=self.g8_ws)
        return F.linear(x, w)

    # Few rows against a long reduction (the decode step's [o | down] projection: K = H*Dv + ff) leave most CUs
    # idle in one GEMM; K is cut into SPLIT_K slices run as one batched GEMM with fp32 partial products, and the
    # residual kernel adds them up (measured 104 -> 35 us at 64 x 25600 -> 4096).
    SPLIT_K, SPLIT_ROWS, SPLIT_MIN_K = 4, 256, 4096

    def _residual_linear(self, x: torch.Tensor, inp: torch.Tensor, w: torch.Tensor) -> None:
        """x (fp32 residual) += m * inp @ w^T."""
        M, K = inp.shape
        S = self.SPLIT_K
        if (self.dtype == torch.bfloat16 and self._split_ok and M <= self.SPLIT_ROWS and K >= self.SPLIT_MIN_K
                and K % (8 * S) == 0):
            parts = torch.bmm(inp.view(M, S, K // S).permute(1, 0, 2), w.view(w.shape[0], S, K // S).permute(1, 2, 0),
                              out_dtype=torch.float32)
            res32.residual_add_partials(x, parts, self.cfg.residual_mult)
            return
        res32.residual_add_scaled(x, self._linear(inp, w), self.cfg.residual_mult)

    def _probe_split(self) -> bool:
        """Whether this torch build runs a bf16 batched GEMM with fp32 output (the split-K path needs it)."""
        if self.dtype != torch.bfloat16:
            return False
        try:
            a = torch.zeros(2, 8, 16, dtype=self.dtype, device=self.device)
            return torch.bmm(a, a.transpose(1, 2), out_dtype=torch.float32).dtype == torch.float32
        except (TypeError, RuntimeError):
            return False

    def tune_gemms(self, M: int, bucket: bool = False, lm_head: bool = True, only=None) -> None:
        """Pick the backend of every projection at M rows by timing the library and the hand-written cores (the
        engine calls this before it captures a decode bucket's graph).  bf16 only, and only where the full kernel
        extension is built; otherwise every GEMM stays on the library."""
        if self.dtype != torch.bfloat16 or only is not None or not ops.available():
            return
        if self.g8_ws is None:
            self.g8_ws = ops.new_gemm8p_workspace(self.device)
        seen = set()
        for L in self.layers:
            for w in (L.w_in, L.w_out):
                if tuple(w.shape) not in seen:
                    seen.add(tuple(w.shape))
                    x = torch.randn(M, w.shape[1], device=self.device).to(self.dtype)
                    gemm_plan.tune(x, w, ws=self.g8_ws, bucket=bucket)
        if lm_head:
            gemm_plan.tune(torch.randn(M, self.cfg.hidden, device=self.device).to(self.dtype), self.head, ws=self.g8_ws,
                           bucket=bucket)

    # ------------------------------------------------------------------ cache
    def _layer_dims(self):
        return [(L.mixer.nk, L.mixer.nv) for L in self.cfg.layer_specs]

    def new_cache(self, num_blocks: int, block_size: int) -> PagedLayerCache:
        return PagedLayerCache(self._layer_dims(), num_blocks, block_size, self.device, self.dtype)

    def bytes_per_block(self, block_size: int) -> int:
        return PagedLayerCache.elems_per_block(self._layer_dims(), block_size) * (4 if self.dtype == torch.float32 else 2)

    # ------------------------------------------------------------------ forward
    def _forward(self, tokens, positions, slots, cache: PagedLayerCache, attend, keep=None, keep_attend=None) -> torch.Tensor:
        """Every layer over the step's rows; ``attend(q, li, out)`` runs the attention of layer ``li`` into
        ``out`` (a column slice).  Returns the fp32 residual stream [T, d].

        ``keep`` (int64 rows; with ``keep_attend``, the attention over just those rows): only these rows' final
        states are wanted (a prompt's last token, a few scored positions).  The LAST layer then still projects
        q | k | v of every row and writes every row's keys and values (later steps read them), but runs the
        attention, the feed-forward and the output projection on the kept rows only; returns [len(keep), d]."""
        cfg = self.cfg
        T = tokens.shape[0]
        x = res32.embed_sinpos(self.embed, tokens, positions, self.inv_freq)
        v0 = None
        nl = len(self.layers)
        for li, (S, L) in enumerate(zip(cfg.layer_specs, self.layers)):
            m = S.mixer
            no, nqkv = m.heads * m.vdim, m.nq + m.nk + m.nv
            short = keep is not None and li + 1 == nl
            h = res32.layernorm(x, L.norm_w, L.norm_b, cfg.norm_eps)
            proj = self._linear(h, L.w_in[:nqkv] if short else L.w_in)
            if L.vmode and v0 is None:
                v0 = torch.empty(T, m.nv, dtype=torch.float32, device=x.device)
            q = res32.proj_norm_kv_write(proj, L.q_norm, L.k_norm, L.head_scale, slots, cache.k[li], cache.v[li],
                                         m.heads, m.dim, cfg.norm_eps, lam=L.vmix, v0=v0, vmode=L.vmode)
            if short:
                x = x.index_select(0, keep)
                cat = torch.empty(keep.numel(), no + S.ff, dtype=self.dtype, device=x.device)
                keep_attend(q.index_select(0, keep), li, cat[:, :no])
                if S.mlp_kind:
                    res32.xielu(self._linear(h.index_select(0, keep), L.w_in[nqkv:]), L.act, cat[:, no:])
            else:
                cat = torch.empty(T, no + S.ff, dtype=self.dtype, device=x.device)
                attend(q, li, cat[:, :no])
                if S.mlp_kind:
                    res32.xielu(proj[:, nqkv:], L.act, cat[:, no:])
            self._residual_linear(x, cat, L.w_out)
            if self.on_layer is not None:
                self.on_layer(li, x)
        return x

    def _logits(self, x: torch.Tensor, rows: Optional[torch.Tensor], float_logits: bool) -> torch.Tensor:
        h = res32.layernorm(x, self.final_w, self.final_b, self.cfg.norm_eps, rows=rows)
        lg = self._linear(h, self.head).float() * self.cfg.logit_scale
        if float_logits:
            return lg
        V, Vp = self.cfg.vocab_size, self.logit_width
        if Vp == V:
            return lg.to(torch.bfloat16)
        out = torch.full((lg.shape[0], Vp), float("-inf"), dtype=torch.bfloat16, device=lg.device)
        out[:, :V] = lg
        return out

    def _attend(self, cache, positions, tables, cu_q=None, k_lens=None, max_q=0):
        def run(q, li, out, rows=slice(None)):
            m = self.cfg.layer_specs[li].mixer
            L = self.layers[li]
            res32.window_attn(q[rows], cache.k[li], cache.v[li], positions[rows], tables, L.r1, L.r2, m.window,
                              out[rows], m.heads, m.kv_heads, cu_q=cu_q, k_lens=k_lens, max_q=max_q, bias=L.bias)
        return run

    def decode(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, block_tables: torch.Tensor,
               ctx_lens: torch.Tensor, cache: PagedLayerCache, num_splits: int = 1, cascade_tiles=None,
               float_logits: bool = False) -> torch.Tensor:
        """One decode step for B sequences -> logits [B, V]; device tensors only (hipGraph-capturable).  Row b
        reads table row b; its key range ends at its own position."""
        x = self._forward(tokens, positions, slots, cache, self._attend(cache, positions, block_tables))
        return self._logits(x, None, float_logits)

    def forward_mixed(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, cache: PagedLayerCache,
                      n_dec: int, dec: Optional[dict], chunk: Optional[dict], logit_rows: torch.Tensor,
                      float_logits: bool = False) -> torch.Tensor:
        """ONE forward over [n_dec decode rows || prompt-portion rows]: every projection is one GEMM over both;
        the attention runs per part (decode rows: table row = row; portion rows: the item of ``chunk['cu_q']``),
        both over the paged cache that this step's rows were just written to.  Logits of ``logit_rows``."""
        T = tokens.shape[0]
        dec_run = self._attend(cache, positions, dec["block_tables"]) if n_dec else None
        chk_run = (self._attend(cache, positions, chunk["block_tables"], cu_q=chunk["cu_q"], k_lens=chunk.get("k_lens"),
                                max_q=int(chunk.get("max_q", 0))) if T > n_dec else None)
        # (the portion rows' cu_q counts from the first portion row: each part gets its own row slice)

        def attend(q, li, out):
            if dec_run is not None:
                dec_run(q, li, out, slice(0, n_dec))
            if chk_run is not None:
                chk_run(q, li, out, slice(n_dec, T))

        # prompt portions of which few rows are wanted (a prompt's last token): the last layer on those rows only
        keep = keep_attend = None
        if n_dec == 0 and self.on_layer is None and 4 * logit_rows.numel() <= T:
            keep = logit_rows
            item = torch.bucketize(logit_rows, chunk["cu_q"][1:].to(torch.int64), right=True)
            keep_attend = self._attend(cache, positions.index_select(0, logit_rows),
                                       chunk["block_tables"].index_select(0, item))
        x = self._forward(tokens, positions, slots, cache, attend, keep=keep, keep_attend=keep_attend)
        return self._logits(x, None if keep is not None else logit_rows, float_logits)

    def prefill(self, tokens, positions, slots, cu_seqlens, max_seqlen, last_idx, cache, ctx=None):
        raise RuntimeError("Madipel prefills through forward_mixed over the paged cache (paged_prefill)")
