"""One MiniMax-M2 decoder block over the raw-block operators: the callers either side of the quantized matmul path.

Host-side mirror of the reference's src/models/minimax_m2/architecture.py (RMSNorm 57-85, MiniMaxAttention 88-268,
MiniMaxMoE 271-385, MiniMaxBlock 388-413): same class names, constructor arguments and call shapes, so that a runtime
written against the reference composes these the same way.  What differs is what runs underneath:

  * the projections are QuantizedGGUFLinear modules of this package (raw GGUF blocks, HIP kernels); q, k and v of a
    decode step leave in ONE launch (gguf_quant_gemm_multi_forward) when the three tensors share a format;
  * routing (gate matvec, sigmoid, bias, top-k, renormalisation) is one operator (moe_route) instead of five framework ops;
  * the experts run through gguf_moe_single_token_forward (one token) or moe_group_routes +
    gguf_moe_prefill_grouped_forward (several tokens), any of the supported expert format pairs.

The attention core itself (rotary embedding, key/value cache, softmax) is not part of the quantized matmul path and stays
framework code, as in the reference (architecture.py:158-266).  One GPU: no tensor-parallel reduction.  The native library
is mandatory; nothing here falls back to a CPU path.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from pocketllm_amd import codebooks
from pocketllm_amd.cuda_loader import load_cuda_kernel
from pocketllm_amd.quantized_ops import QuantizedGGUFLinear
from pocketllm_amd.quantized_tensor import QuantizedGGUFTensor


@dataclass(frozen=True)
class MiniMaxM2Args:
    """The fields of the reference's MiniMaxM2Args (architecture.py:19-34) that a block reads."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    rope_dim: int
    rope_base: float
    n_routed_experts: int
    top_k: int
    moe_inter_dim: int
    norm_eps: float


def _kernel():
    mod = load_cuda_kernel()
    if mod is None:
        raise RuntimeError("the native HIP library is required for the MiniMax block")
    return mod


class RMSNorm:
    """architecture.py:57-85: the fused normalisation operator, fp16 output."""

    def __init__(self, weight: torch.Tensor, eps: float, *, out_dtype: torch.dtype = torch.float16):
        self.weight = weight.float().contiguous()
        self.eps = float(eps)
        self.out_dtype = out_dtype
        self._cuda = _kernel()

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        x_flat = x.reshape(-1, x.size(-1)).contiguous()
        return self._cuda.fused_rms_norm_forward(x_flat, self.weight, self.eps).view(x.shape).to(self.out_dtype)


@dataclass
class ExpertLayer:
    """The three routed tensors of one layer, [experts, rows, blocks per row, block bytes] each (what the reference's
    device-resident cache hands out per layer, moe_runtime.py:175-188)."""
    w1: QuantizedGGUFTensor
    w3: QuantizedGGUFTensor
    w2: QuantizedGGUFTensor


class MiniMaxMoE:
    """architecture.py:271-385 on one GPU: route, then the fused experts."""

    def __init__(self, args: MiniMaxM2Args, gate_weight: torch.Tensor, gate_bias: torch.Tensor | None, experts: ExpertLayer,
                 *, expert_start: int = 0, dtype: torch.dtype = torch.float16):
        self.args = args
        self.gate_weight = gate_weight.float().contiguous()
        self.gate_bias = gate_bias.float().contiguous() if gate_bias is not None else None
        self.experts = experts
        self.expert_start = int(expert_start)
        self.expert_count = int(experts.w1.blocks.size(0))
        self.dtype = dtype
        self._cuda = _kernel()
        dev = experts.w1.blocks.device
        ids = {int(experts.w1.type_id), int(experts.w3.type_id), int(experts.w2.type_id)}
        # the grid argument of the reference's operators: one codebook, or the pair when gate/up and down use different ones
        grids = [codebooks.grid_tensor_for_type(t).to(dev) for t in sorted(ids) if t in (0, 2)]
        self._grid = grids[0] if len(grids) == 1 else (tuple(grids) if grids else torch.empty(0, dtype=torch.int8, device=dev))

    def route(self, x_flat: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """architecture.py:291-298 as one operator: sigmoid scores, bias for the selection only, top-k, renormalised weights."""
        return self._cuda.moe_route(x_flat, self.gate_weight, self.gate_bias, int(self.args.top_k))

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        original_shape = x.shape
        x_flat = x.reshape(-1, original_shape[-1]).contiguous()
        indices, weights = self.route(x_flat)
        e = self.experts
        if x_flat.size(0) == 1:
            slots = indices[0]
            local = (slots >= self.expert_start) & (slots < self.expert_start + self.expert_count)
            if self.expert_start == 0 and self.expert_count >= int(self.args.n_routed_experts):
                local_slots, local_weights = slots, weights[0]                 # every expert is resident: nothing to filter
            else:
                local_slots, local_weights = slots[local] - self.expert_start, weights[0][local]
            if local_slots.numel() == 0:
                y = torch.zeros((1, self.args.dim), device=x.device, dtype=torch.float32)
            else:
                y = self._cuda.gguf_moe_single_token_forward(x_flat, local_slots.contiguous(), local_weights.contiguous(),
                                                             e.w1.blocks, e.w3.blocks, e.w2.blocks, 0.0)
        else:
            _ids, route_tokens, route_weights, seg = self._cuda.moe_group_routes(indices, weights, self.expert_start, self.expert_count)
            if int(route_tokens.numel()) == 0:
                y = torch.zeros((x_flat.size(0), self.args.dim), device=x.device, dtype=torch.float32)
            else:
                y = self._cuda.gguf_moe_prefill_grouped_forward(
                    x_flat, route_tokens, route_weights, seg, e.w1.blocks, e.w3.blocks, e.w2.blocks,
                    int(e.w1.row_elems), int(e.w1.type_id), int(e.w3.row_elems), int(e.w3.type_id), int(e.w2.row_elems), int(e.w2.type_id),
                    self._grid, 0.0)
        return y.reshape(original_shape).to(self.dtype)


class MiniMaxAttention:
    """architecture.py:88-268: q / k / v projections, per-projection RMS normalisation of q and k, half-split rotary embedding
    over the first rope_dim values of every head, key/value cache, scaled dot-product attention, output projection."""

    def __init__(self, args: MiniMaxM2Args, q_proj: QuantizedGGUFLinear, k_proj: QuantizedGGUFLinear, v_proj: QuantizedGGUFLinear,
                 o_proj: QuantizedGGUFLinear, q_norm: RMSNorm, k_norm: RMSNorm, *, dtype: torch.dtype = torch.float16):
        self.args = args
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = q_proj, k_proj, v_proj, o_proj
        self.q_norm, self.k_norm = q_norm, k_norm
        self.dtype = dtype
        self.cache_k: torch.Tensor | None = None
        self.cache_v: torch.Tensor | None = None
        self._cuda = _kernel()
        tensors = (q_proj.tensor, k_proj.tensor, v_proj.tensor)
        self._one_launch = len({int(t.type_id) for t in tensors}) == 1 and len({int(t.blocks.size(1)) for t in tensors}) == 1 \
            and int(tensors[0].type_id) != 1

    def reset_cache(self, batch_size: int, max_seq_len: int) -> None:
        dev = self.q_proj.tensor.blocks.device
        shape = (batch_size, max_seq_len, self.args.n_kv_heads, self.args.head_dim)
        self.cache_k = torch.zeros(shape, device=dev, dtype=self.dtype)
        self.cache_v = torch.zeros(shape, device=dev, dtype=self.dtype)

    def _apply_rope(self, x: torch.Tensor, start_pos: int) -> torch.Tensor:
        rope_dim = int(self.args.rope_dim)
        if rope_dim <= 0:
            return x
        half = rope_dim // 2
        positions = torch.arange(start_pos, start_pos + x.size(1), device=x.device, dtype=torch.float32)
        j = torch.arange(half, device=x.device, dtype=torch.float32)
        inv = torch.pow(torch.full_like(j, float(self.args.rope_base)), -(2.0 * j) / float(rope_dim))
        freqs = positions[:, None] * inv[None, :]
        sin = torch.sin(freqs).to(x.dtype)[None, :, None, :]
        cos = torch.cos(freqs).to(x.dtype)[None, :, None, :]
        x1, x2 = x[..., :half], x[..., half:rope_dim]
        parts = [x1 * cos - x2 * sin, x1 * sin + x2 * cos]
        if rope_dim < x.size(-1):
            parts.append(x[..., rope_dim:])
        return torch.cat(parts, dim=-1)

    def _qkv(self, x: torch.Tensor):
        rows = x.numel() // x.size(-1)
        if self._one_launch and rows <= 4:                  # decode: the three projections of one activation row as one launch
            t = self.q_proj.tensor
            q, k, v = self._cuda.gguf_quant_gemm_multi_forward(
                x.contiguous(), (self.q_proj.tensor.blocks, self.k_proj.tensor.blocks, self.v_proj.tensor.blocks), int(t.row_elems),
                int(t.type_id), self.q_proj._grid, out_dtype=self.dtype)
            return q, k, v
        return self.q_proj(x), self.k_proj(x), self.v_proj(x)

    def __call__(self, x: torch.Tensor, start_pos: int) -> torch.Tensor:
        bsz, seqlen, _ = x.shape
        end_pos = int(start_pos) + int(seqlen)
        if self.cache_k is None or self.cache_k.size(0) < bsz or self.cache_k.size(1) < end_pos:
            self.reset_cache(bsz, max(end_pos, 256))
        a = self.args
        q_raw, k_raw, v_raw = self._qkv(x)
        q = self.q_norm(q_raw).view(bsz, seqlen, a.n_heads, a.head_dim)
        k = self.k_norm(k_raw).view(bsz, seqlen, a.n_kv_heads, a.head_dim)
        v = v_raw.view(bsz, seqlen, a.n_kv_heads, a.head_dim).to(self.dtype)
        q = self._apply_rope(q, int(start_pos))
        k = self._apply_rope(k, int(start_pos))
        self.cache_k[:bsz, start_pos:end_pos].copy_(k)
        self.cache_v[:bsz, start_pos:end_pos].copy_(v)
        q_t = q.transpose(1, 2).contiguous()
        k_t = self.cache_k[:bsz, :end_pos].transpose(1, 2).contiguous()
        v_t = self.cache_v[:bsz, :end_pos].transpose(1, 2).contiguous()
        repeat = a.n_heads // a.n_kv_heads
        if repeat != 1:
            k_t = k_t.repeat_interleave(repeat, dim=1)
            v_t = v_t.repeat_interleave(repeat, dim=1)
        mask, causal = None, False
        if seqlen > 1 and int(start_pos) == 0:
            causal = True
        elif seqlen > 1:
            q_pos = torch.arange(start_pos, end_pos, device=x.device)
            k_pos = torch.arange(0, end_pos, device=x.device)
            mask = torch.zeros((seqlen, end_pos), device=x.device, dtype=q_t.dtype)
            mask.masked_fill_(~(k_pos[None, :] <= q_pos[:, None]), float("-inf"))
        out = F.scaled_dot_product_attention(q_t.to(self.dtype), k_t.to(self.dtype), v_t.to(self.dtype), attn_mask=mask, dropout_p=0.0,
                                             is_causal=causal, scale=1.0 / math.sqrt(float(a.head_dim)))
        out = out.transpose(1, 2).contiguous().view(bsz, seqlen, a.n_heads * a.head_dim)
        return self.o_proj(out)


class MiniMaxBlock:
    """architecture.py:388-413: x + attention(norm(x)), then x + experts(norm(x)), each sum rounded to the model's dtype."""

    def __init__(self, args: MiniMaxM2Args, attn_norm_weight: torch.Tensor, ffn_norm_weight: torch.Tensor, attention: MiniMaxAttention,
                 moe: MiniMaxMoE, *, dtype: torch.dtype = torch.float16):
        self.args = args
        self.attn_norm = RMSNorm(attn_norm_weight, args.norm_eps, out_dtype=dtype)
        self.ffn_norm = RMSNorm(ffn_norm_weight, args.norm_eps, out_dtype=dtype)
        self.attention = attention
        self.moe = moe
        self.dtype = dtype

    def reset_cache(self, batch_size: int, max_seq_len: int) -> None:
        self.attention.reset_cache(batch_size, max_seq_len)

    def __call__(self, x: torch.Tensor, start_pos: int) -> torch.Tensor:
        x = (x + self.attention(self.attn_norm(x), start_pos)).to(self.dtype)
        x = (x + self.moe(self.ffn_norm(x))).to(self.dtype)
        return x
