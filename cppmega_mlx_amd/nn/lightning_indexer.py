"""Lightning indexer: which KV positions each query attends to.

Surface of the reference's ``cppmega_v4/nn/lightning_indexer.py`` (``LightningIndexerConfig``
:23-44, ``_apply_non_interleaved_rope`` :47-79, ``LightningIndexer`` :82-145) and of its FP8
variant ``cppmega_v4/nn/lightning_indexer_fp8.py`` (``LightningIndexerFP8Config`` :54-58,
``LightningIndexerFP8`` :61-157): ``indexer(x, qr, (cos, sin), mask=None) -> int32 [B, T, topk]``.

The score-and-select tail (:132-145) is the HIP path: ``ops.indexer_topk`` forms the head-weighted
query, multiplies it with the key rows on the matrix cores and hands the scores to the radix
selector without keeping the [B, T, T_kv] matrix.  ``indexer_scores_topk`` exposes that tail on its
own for callers that already hold q, k and the head weights.  The small projections in front of it
(wq_b, wk, LayerNorm, weights_proj, rope) are torch tensor operations here, except the FP8
variant's wq_b, which runs the block-128 FP8 kernel on the stored bytes instead of dequantising
the weight first.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import ops
from ._tilelang.fused_fp8_gemm import fused_fp8_gemm

__all__ = [
    "LightningIndexer",
    "LightningIndexerConfig",
    "LightningIndexerFP8",
    "LightningIndexerFP8Config",
    "indexer_scores_topk",
    "quantize_indexer_weights_for_fp8",
]


@dataclass(frozen=True)
class LightningIndexerConfig:
    hidden_size: int
    n_heads: int
    head_dim: int = 32
    rope_head_dim: int = 16
    q_lora_rank: int = 1536
    index_topk: int = 64
    softmax_scale: float | None = None
    norm_eps: float = 1e-6

    def __post_init__(self) -> None:
        if self.head_dim <= 0 or self.rope_head_dim <= 0:
            raise ValueError("head_dim and rope_head_dim must be positive")
        if self.rope_head_dim > self.head_dim:
            raise ValueError("rope_head_dim must be <= head_dim")
        if self.n_heads <= 0:
            raise ValueError("n_heads must be positive")
        if self.index_topk <= 0:
            raise ValueError("index_topk must be positive")


@dataclass(frozen=True)
class LightningIndexerFP8Config(LightningIndexerConfig):
    fp8_blocks: bool = True


def _apply_non_interleaved_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate the halves (x[..., :d], x[..., d:]) as planes; cos/sin are (T, d), T on axis 1 of x."""
    if x.shape[-1] % 2 != 0:
        raise ValueError(f"rope dim must be even, got {x.shape[-1]}")
    d = x.shape[-1] // 2
    x1, x2 = x[..., :d], x[..., d:]
    cos_b, sin_b = cos.to(x.dtype), sin.to(x.dtype)
    if x.ndim > 2:
        shape = (1, cos_b.shape[0]) + (1,) * (x.ndim - 3) + (cos_b.shape[1],)
        cos_b, sin_b = cos_b.reshape(shape), sin_b.reshape(shape)
    return torch.cat([x1 * cos_b - x2 * sin_b, x2 * cos_b + x1 * sin_b], dim=-1)


def indexer_scores_topk(q: torch.Tensor, k: torch.Tensor, weights: torch.Tensor, *, sm_scale: float, index_topk: int,
                        mask: torch.Tensor | None = None, ends: torch.Tensor | None = None,
                        out: torch.Tensor | None = None) -> torch.Tensor:
    """``argpartition(-(einsum("bqhd,bkd,bqh->bqk") * sm_scale + mask))[..., :topk]`` as int32
    [B, T, min(index_topk, T_kv)], ascending by index; ``ends`` ([B*T] int32) bounds each row's
    selectable keys without a mask read."""
    B, T = q.shape[0], q.shape[1]
    topk = min(int(index_topk), int(k.shape[1]))
    if out is None:
        out = torch.empty((B, T, topk), dtype=torch.int32, device=q.device)
    return ops.indexer_topk(q.contiguous(), k.contiguous(), weights.contiguous(), sm_scale=sm_scale, topk=topk, out=out,
                            mask=None if mask is None else mask.contiguous(), ends=ends)


def _layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), weight.to(x.dtype), bias.to(x.dtype), eps)


class LightningIndexer:
    """fp32/bf16 indexer: ``__call__(x [B,T,hidden], qr [B,T,q_lora_rank], (cos, sin), mask=None)``."""

    def __init__(self, config: LightningIndexerConfig, *, device=None, dtype: torch.dtype = torch.float32, seed: int = 0):
        self.config = config
        gen = torch.Generator(device="cpu").manual_seed(seed)

        def init(out_f: int, in_f: int) -> torch.Tensor:
            bound = in_f ** -0.5
            return ((torch.rand((out_f, in_f), generator=gen) * 2 - 1) * bound).to(device=device, dtype=dtype)

        self.wq_b = init(config.n_heads * config.head_dim, config.q_lora_rank)
        self.wk = init(config.head_dim, config.hidden_size)
        self.weights_proj = init(config.n_heads, config.hidden_size)
        self.k_norm_weight = torch.ones(config.head_dim, device=device, dtype=dtype)
        self.k_norm_bias = torch.zeros(config.head_dim, device=device, dtype=dtype)

    def _project_q(self, qr: torch.Tensor) -> torch.Tensor:
        return qr @ self.wq_b.T

    def _prepare(self, x: torch.Tensor, qr: torch.Tensor, freqs_cis):
        cfg = self.config
        batch, seq, _ = x.shape
        cos, sin = freqs_cis
        q = self._project_q(qr).reshape(batch, seq, cfg.n_heads, cfg.head_dim)
        q = torch.cat([_apply_non_interleaved_rope(q[..., : cfg.rope_head_dim], cos, sin), q[..., cfg.rope_head_dim:]], dim=-1)
        k = _layer_norm(x @ self.wk.T.to(x.dtype), self.k_norm_weight, self.k_norm_bias, cfg.norm_eps)
        k = torch.cat([_apply_non_interleaved_rope(k[..., : cfg.rope_head_dim], cos, sin), k[..., cfg.rope_head_dim:]], dim=-1)
        weights = (x @ self.weights_proj.T.to(x.dtype)) * (cfg.n_heads ** -0.5)
        sm_scale = cfg.softmax_scale if cfg.softmax_scale is not None else cfg.head_dim ** -0.5
        return q, k, weights, sm_scale

    def __call__(self, x: torch.Tensor, qr: torch.Tensor, freqs_cis, mask: torch.Tensor | None = None) -> torch.Tensor:
        q, k, weights, sm_scale = self._prepare(x, qr, freqs_cis)
        carrier = torch.bfloat16 if q.dtype == torch.bfloat16 else torch.float32
        return indexer_scores_topk(q.to(carrier), k.to(carrier), weights.to(carrier), sm_scale=sm_scale,
                                   index_topk=self.config.index_topk, mask=mask)


class LightningIndexerFP8(LightningIndexer):
    """The indexer with ``wq_b`` stored as e4m3 bytes + one float32 scale per 128x128 block; q, k
    and the head weights are bfloat16."""

    def __init__(self, config: LightningIndexerFP8Config, *, device=None, seed: int = 0):
        super().__init__(config, device=device, dtype=torch.bfloat16, seed=seed)
        out_dim = config.n_heads * config.head_dim
        if config.fp8_blocks:
            self._wq_b_fp8 = torch.zeros((out_dim, config.q_lora_rank), dtype=torch.uint8, device=device)
            self._wq_b_scale_inv = torch.ones(((out_dim + 127) // 128, (config.q_lora_rank + 127) // 128),
                                              dtype=torch.float32, device=device)

    def _project_q(self, qr: torch.Tensor) -> torch.Tensor:
        if self.config.fp8_blocks:
            return fused_fp8_gemm(self._wq_b_fp8, self._wq_b_scale_inv, qr.to(torch.bfloat16).contiguous())
        return qr.to(torch.bfloat16) @ self.wq_b.T

    def load_fp8_weights(self, wq_b_fp8, wq_b_scale_inv, wk_bf16, weights_proj_bf16, k_norm_weight=None, k_norm_bias=None) -> None:
        if not self.config.fp8_blocks:
            raise AssertionError("load_fp8_weights requires fp8_blocks=True")
        if wq_b_fp8.dtype != torch.uint8:
            raise TypeError(f"wq_b_fp8 must be uint8 (fp8 storage); got {wq_b_fp8.dtype}")
        self._wq_b_fp8 = wq_b_fp8.contiguous()
        self._wq_b_scale_inv = wq_b_scale_inv.to(torch.float32).contiguous()
        self.wk = wk_bf16.to(torch.bfloat16)
        self.weights_proj = weights_proj_bf16.to(torch.bfloat16)
        if k_norm_weight is not None:
            self.k_norm_weight = k_norm_weight.to(torch.bfloat16)
        if k_norm_bias is not None:
            self.k_norm_bias = k_norm_bias.to(torch.bfloat16)

    def __call__(self, x: torch.Tensor, qr: torch.Tensor, freqs_cis, mask: torch.Tensor | None = None) -> torch.Tensor:
        return super().__call__(x.to(torch.bfloat16), qr, freqs_cis, mask)


def quantize_indexer_weights_for_fp8(indexer: LightningIndexer) -> dict[str, torch.Tensor | None]:
    """Checkpoint tensors ``LightningIndexerFP8.load_fp8_weights`` accepts, from a float indexer
    (reference: lightning_indexer_fp8.py:160-197): ``wq_b`` as e4m3 bytes with one
    ``amax / 448`` float32 scale per 128x128 block (amax floored at 1e-6), the scaled values
    passing through bfloat16 on the way to e4m3 as in the reference; the rest bfloat16."""
    w = indexer.wq_b.to(torch.float32)
    m, n = w.shape
    pad_m, pad_n = (-m) % 128, (-n) % 128
    padded = torch.nn.functional.pad(w, (0, pad_n, 0, pad_m))
    blocks = padded.reshape((m + pad_m) // 128, 128, (n + pad_n) // 128, 128)
    amax = blocks.abs().amax(dim=(1, 3)).clamp_min(1e-6)
    scale_inv = (amax / 448.0).to(torch.float32)
    scaled = (blocks / scale_inv[:, None, :, None]).reshape(m + pad_m, n + pad_n)[:m, :n]
    codes = scaled.to(torch.bfloat16).float().clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    return {
        "wq_b_fp8": codes.contiguous(),
        "wq_b_scale_inv": scale_inv.contiguous(),
        "wk_bf16": indexer.wk.to(torch.bfloat16),
        "weights_proj_bf16": indexer.weights_proj.to(torch.bfloat16),
        "k_norm_weight": indexer.k_norm_weight.to(torch.bfloat16),
        "k_norm_bias": indexer.k_norm_bias.to(torch.bfloat16),
    }
