"""Python face of the fp32-residual kernel set (``csrc/kernels/res32`` -> ``ops/_res32.so``).

For decoder designs that keep their residual stream, norms, attention scores and cache-write arithmetic in fp32
while the activations between kernels are bf16 (serving) or fp32 (exact mode).  The extension is separate from
``_kernels.so`` so that a model of such a design needs only this one built; it is compiled on first use when
missing (a fresh checkout), and there is no eager-PyTorch fallback.

Cache layout shared with :class:`..models.cache.PagedLayerCache`: per layer K ``[num_blocks, block_size, G*D]``
and V ``[num_blocks, block_size/4, G*Dv, 4]`` (4-token interleaved) as strided views of one pool.
"""
from __future__ import annotations

import importlib
import math
import threading
from typing import Optional

import torch

_K = None
_LOCK = threading.Lock()


def kernels():
    """The loaded ``_res32`` extension; built in-tree first when it is not there."""
    global _K
    if _K is None:
        with _LOCK:
            if _K is None:
                try:
                    _K = importlib.import_module("llm_weighted_consensus_amd.ops._res32")
                except ImportError:
                    from .. import _build

                    _build.build_res32()
                    _K = importlib.import_module("llm_weighted_consensus_amd.ops._res32")
    return _K


def sinpos_inv_freq(d: int, base: float = 10000.0, device="cuda") -> torch.Tensor:
    """base^(-2i/d) for i < ceil(d/2), in float64 (the kernel reduces p * f mod 2 pi in double)."""
    i2 = torch.arange(0, d, 2, dtype=torch.float64)
    return (float(base) ** (-i2 / d)).to(device)


def embed_sinpos(table: torch.Tensor, tokens: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[t] = table[tokens[t]] + s(positions[t]) in fp32, s[2i] = sin(p f_i), s[2i+1] = cos(p f_i)."""
    if out is None:
        out = torch.empty(tokens.numel(), table.shape[1], dtype=torch.float32, device=table.device)
    kernels().embed_sinpos(table, tokens, positions, inv_freq, out)
    return out


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm with weight and bias of fp32 rows (statistics in fp32) -> rows of ``w``'s dtype.  ``rows``
    (int64): normalise only these rows of ``x``, in this order."""
    n = x.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty(n, x.shape[1], dtype=w.dtype, device=x.device)
    kernels().layernorm(x, rows, w, b, out, float(eps))
    return out


def proj_norm_kv_write(proj: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, head_scale: torch.Tensor,
                       slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, D: int, eps: float,
                       lam: Optional[torch.Tensor] = None, v0: Optional[torch.Tensor] = None, vmode: int = 0,
                       q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From fused projection rows ``[q | k | v | ...]``: q and k each RMS-normalised over their whole projection
    (all heads at once) with plain weights; q scaled per head by ``head_scale`` into an fp32 buffer (returned);
    k and v written into the paged cache at ``slots`` (-1: no write).  ``vmode`` 1 publishes v into ``v0``
    (fp32 [T, nv]); 2 blends v <- (1 - lam) v + lam v0 before the cache write."""
    if q_out is None:
        q_out = torch.empty(proj.shape[0], H * D, dtype=torch.float32, device=proj.device)
    kernels().proj_norm_kv_write(proj, wq, wk, head_scale, lam, v0, int(vmode), slots, q_out, k_cache, v_cache,
                                 int(H), int(D), float(eps))
    return q_out


def xielu(z: torch.Tensor, pq: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """xIELU with the two raw parameters ``pq`` = (p, q): z > 0: softplus(p) z^2 + z/2; else
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2.  ``z`` and ``out`` may be column slices of wider row-dense buffers."""
    kernels().xielu(z, pq, out)
    return out


def residual_add_scaled(x: torch.Tensor, y: torch.Tensor, m: float) -> None:
    """x (fp32) += m * y, in place."""
    kernels().residual_add_scaled(x, y, float(m))


def residual_add_partials(x: torch.Tensor, parts: torch.Tensor, m: float) -> None:
    """x (fp32) += m * parts.sum(0), parts fp32 [S, *x.shape] (the partial products of a split-K GEMM)."""
    kernels().residual_add_partials(x, parts, float(m))


def distance_bias(r1: torch.Tensor, r2: torch.Tensor, window: int) -> torch.Tensor:
    """The table b[h, n] = r1_h ln(1 + r2_h n), n < window (fp32), that the matrix-core kernel reads."""
    n = torch.arange(window, dtype=torch.float32, device=r1.device)
    return (r1.float()[:, None] * torch.log1p(r2.float()[:, None] * n[None, :])).contiguous()


def window_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, positions: torch.Tensor,
                block_tables: torch.Tensor, r1: torch.Tensor, r2: torch.Tensor, window: int, out: torch.Tensor,
                H: int, G: int, cu_q: Optional[torch.Tensor] = None, k_lens: Optional[torch.Tensor] = None,
                max_q: int = 0, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sliding-window attention over the paged cache with the bias -r1_h ln(1 + r2_h (i - j)); ``q`` fp32
    [T, H*D] pre-scaled; row t reads table row t (``cu_q`` None) or the item whose ``cu_q`` range holds t.
    Over a bf16 cache whose sizes the matrix-core kernels are built for, prompt portions run on the portion kernel
    (it wants ``k_lens``, ``max_q`` and the ``bias`` table of :func:`distance_bias`) and decode rows on the
    split-key decode kernel (``bias``); everything else on the general kernel."""
    K = kernels()
    bs = k_cache.shape[1]
    cores = (bias is not None and k_cache.dtype == torch.bfloat16 and bs & (bs - 1) == 0
             and K.window_attn_mfma_ok(k_cache.shape[2] // G, v_cache.shape[2] // G))
    if cores and cu_q is None and positions.numel() > 0:
        max_keys = min(int(window), block_tables.shape[1] * k_cache.shape[1])
        K.window_attn_decode(q, k_cache, v_cache, positions, block_tables, bias, int(window), max_keys, out, int(H), int(G))
        return out
    if cores and cu_q is not None and k_lens is not None and max_q > 0:
        K.window_attn_mfma(q, k_cache, v_cache, positions, cu_q, k_lens, int(max_q), block_tables, bias, int(window), out,
                           int(H), int(G))
        return out
    K.window_attn(q, k_cache, v_cache, positions, cu_q, block_tables, r1, r2, int(window), out, int(H), int(G))
    return out


def softplus(x: float) -> float:
    return max(x, 0.0) + math.log1p(math.exp(-abs(x)))
