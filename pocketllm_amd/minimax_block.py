"""One MiniMax-M2 decoder block over the raw-block operators: the callers either side of the quantized matmul path.

Host-side mirror of the reference's src/models/minimax_m2/architecture.py (RMSNorm 57-85, MiniMaxAttention 88-268,
MiniMaxMoE 271-385, MiniMaxBlock 388-413, MiniMaxTransformer 417-472): same class names, constructor arguments and call
shapes, so that a runtime written against the reference composes these the same way.  What differs is what runs underneath:

  * the projections are QuantizedGGUFLinear modules of this package (raw GGUF blocks, HIP kernels); q, k and v of a
    decode step leave in ONE launch (gguf_quant_gemm_multi_forward) when the three tensors share a format;
  * routing (gate matvec, sigmoid, bias, top-k, renormalisation) is one operator (moe_route) instead of five framework ops;
  * the experts run through gguf_moe_single_token_forward (one token) or moe_group_routes +
    gguf_moe_prefill_grouped_forward (several tokens), any of the supported expert format pairs;
  * a decode step folds both residual connections and both normalisations it can into the projections: the block's first
    RMS normalisation runs inside the q / k / v launch, the output projection adds into the residual stream in its store.

The attention core itself (rotary phases, key/value store, softmax) is not part of the quantized matmul path; it lives in
attention_core.py as plain framework arithmetic of this package's own (head-major cache, grouped matrix products, float32
softmax).  One GPU: no tensor-parallel reduction.  The native library is mandatory; nothing here falls back to a CPU path.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from pocketllm_amd import codebooks
from pocketllm_amd.attention_core import KeyValueCache, RotaryTable, grouped_query_attention
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
        rows = x.contiguous().view(-1, x.size(-1))
        return self._cuda.fused_rms_norm_forward(rows, self.weight, self.eps, out_dtype=self.out_dtype).view(x.shape)


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

    def __call__(self, x: torch.Tensor, residual: torch.Tensor | None = None, input_norm: RMSNorm | None = None) -> torch.Tensor:
        """The experts' output for x in the model's dtype; with `residual` (x's shape, the model's dtype) it is added into that
        tensor, which is returned.  `input_norm`, when given, is the block's normalisation of the residual stream: the experts see
        input_norm(x), and decode steps run it inside the routing launch."""
        tokens = x.reshape(-1, x.size(-1)).contiguous()
        routed = None
        if input_norm is not None:
            if tokens.size(0) <= 4:
                routed = self._cuda.moe_route_rmsnorm(tokens, input_norm.weight, input_norm.eps, self.gate_weight, self.gate_bias,
                                                      int(self.args.top_k), out_dtype=input_norm.out_dtype)
            if routed is None:
                tokens = input_norm(tokens)
        if routed is not None:
            chosen, gate_w, tokens = routed
        else:
            chosen, gate_w = self.route(tokens)
        w = self.experts
        nothing = lambda: tokens.new_zeros((tokens.size(0), self.args.dim), dtype=torch.float32)   # no route lands on a resident expert
        if tokens.size(0) == 1:
            ids, ws = chosen[0], gate_w[0]
            if not (self.expert_start == 0 and self.expert_count >= int(self.args.n_routed_experts)):   # a slice of the experts is resident
                here = (ids >= self.expert_start) & (ids < self.expert_start + self.expert_count)
                ids, ws = ids[here] - self.expert_start, ws[here]
            if ids.numel() == 0:
                out = nothing()
            else:
                # the down projection adds the routes' sum into the residual stream itself where it has a kernel for it
                if residual is not None and residual.is_contiguous() and self._cuda.gguf_moe_single_token_accumulate_forward(
                        tokens, ids.contiguous(), ws.contiguous(), w.w1.blocks, w.w3.blocks, w.w2.blocks, 0.0, residual):
                    return residual
                out = self._cuda.gguf_moe_single_token_forward(tokens, ids.contiguous(), ws.contiguous(), w.w1.blocks, w.w3.blocks, w.w2.blocks, 0.0)
        else:
            _, route_tokens, route_weights, seg = self._cuda.moe_group_routes(chosen, gate_w, self.expert_start, self.expert_count)
            out = nothing() if route_tokens.numel() == 0 else self._cuda.gguf_moe_prefill_grouped_forward(
                tokens, route_tokens, route_weights, seg, w.w1.blocks, w.w3.blocks, w.w2.blocks,
                int(w.w1.row_elems), int(w.w1.type_id), int(w.w3.row_elems), int(w.w3.type_id), int(w.w2.row_elems), int(w.w2.type_id), self._grid, 0.0)
        y = out.view(x.shape).to(self.dtype)
        return y if residual is None else residual.add_(y)


class MiniMaxAttention:
    """The attention half of a block (reference: architecture.py:88-268): q / k / v projections, RMS normalisation of q and k
    over the whole projection width, rotary phases on the first rope_dim values of every head, key/value store, grouped-query
    softmax attention, output projection.  `input_norm`, when given, is the block's normalisation of the residual stream: decode
    steps then run it inside the q / k / v launch."""

    def __init__(self, args: MiniMaxM2Args, q_proj: QuantizedGGUFLinear, k_proj: QuantizedGGUFLinear, v_proj: QuantizedGGUFLinear,
                 o_proj: QuantizedGGUFLinear, q_norm: RMSNorm, k_norm: RMSNorm, *, dtype: torch.dtype = torch.float16):
        self.args = args
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = q_proj, k_proj, v_proj, o_proj
        self.q_norm, self.k_norm = q_norm, k_norm
        self.dtype = dtype
        self._cuda = _kernel()
        dev = q_proj.tensor.blocks.device
        self.rotary = RotaryTable(args.rope_dim, args.rope_base, dev, head_dim=args.head_dim)
        self.store = KeyValueCache(args.n_kv_heads, args.head_dim, dev, dtype)
        qkv = (q_proj.tensor, k_proj.tensor, v_proj.tensor)
        # one launch for the three projections needs one format (not Q2_K) and one row length
        self._fused_qkv = len({(int(t.type_id), int(t.blocks.size(1))) for t in qkv}) == 1 and int(qkv[0].type_id) != 1
        # the one-operator decode step: 128-wide heads, groups of up to 8, 16-bit stores, both normalisations with one eps
        self._fused_step = (args.head_dim == 128 and args.n_heads % args.n_kv_heads == 0 and args.n_heads // args.n_kv_heads <= 8 and
                            dtype in (torch.float16, torch.bfloat16) and q_norm.eps == k_norm.eps and self._cuda is not None and dev.type == "cuda")

    def reset_cache(self, batch_size: int, max_seq_len: int) -> None:
        self.store.allocate(batch_size, max_seq_len)
        self.rotary.reserve(max_seq_len)

    def project_qkv(self, x: torch.Tensor, input_norm: RMSNorm | None = None):
        """q, k, v of x [batch, steps, dim] (of input_norm(x) when a normalisation is handed in)."""
        rows = x.numel() // x.size(-1)
        if self._fused_qkv and rows <= 4:
            t = self.q_proj.tensor
            return self._cuda.gguf_quant_gemm_multi_forward(
                x.contiguous(), [p.tensor.blocks for p in (self.q_proj, self.k_proj, self.v_proj)], int(t.row_elems), int(t.type_id),
                self.q_proj._grid, norm_weight=None if input_norm is None else input_norm.weight,
                eps=0.0 if input_norm is None else input_norm.eps, out_dtype=self.dtype)
        h = x if input_norm is None else input_norm(x)
        return self.q_proj(h), self.k_proj(h), self.v_proj(h)

    def context(self, x: torch.Tensor, start_pos: int, input_norm: RMSNorm | None = None) -> torch.Tensor:
        """Everything up to the output projection: [batch, steps, heads * head_dim]."""
        a = self.args
        batch, steps = x.size(0), x.size(1)
        q, k, v = self.project_qkv(x, input_norm)
        if steps == 1 and self._fused_step and start_pos < 131072:
            # a decode step: normalisation, rotary phases, store update and attention in one operator (two launches)
            self.store.ensure(batch, start_pos + 1)
            cos_row, sin_row = self.rotary.rows(start_pos)
            return self._cuda.attention_decode_forward(
                q.view(batch, -1).to(self.dtype), k.view(batch, -1).to(self.dtype), v.view(batch, -1).to(self.dtype), self.store.keys, self.store.values,
                start_pos, q_norm_weight=self.q_norm.weight, k_norm_weight=self.k_norm.weight, eps=self.q_norm.eps, cos_row=cos_row, sin_row=sin_row,
                rope_dim=2 * self.rotary.half).view(batch, 1, -1)
        q = self.rotary.rotate(self.q_norm(q).view(batch, steps, a.n_heads, a.head_dim), start_pos)
        k = self.rotary.rotate(self.k_norm(k).view(batch, steps, a.n_kv_heads, a.head_dim), start_pos)
        self.store.write(k, v.view(batch, steps, a.n_kv_heads, a.head_dim).to(self.dtype), start_pos)
        keys, values = self.store.read(batch, start_pos + steps)
        return grouped_query_attention(q.to(self.dtype), keys, values, start_pos)

    def __call__(self, x: torch.Tensor, start_pos: int) -> torch.Tensor:
        return self.o_proj(self.context(x, int(start_pos)))


class MiniMaxBlock:
    """One decoder layer (reference: architecture.py:388-413): attention and routed experts, each behind an RMS normalisation
    and added back to the residual stream, which is kept in the model's dtype."""

    def __init__(self, args: MiniMaxM2Args, attn_norm_weight: torch.Tensor, ffn_norm_weight: torch.Tensor, attention: MiniMaxAttention,
                 moe: MiniMaxMoE, *, dtype: torch.dtype = torch.float16):
        self.args = args
        self.attn_norm = RMSNorm(attn_norm_weight, args.norm_eps, out_dtype=dtype)
        self.ffn_norm = RMSNorm(ffn_norm_weight, args.norm_eps, out_dtype=dtype)
        self.attention = attention
        self.moe = moe
        self.dtype = dtype
        self._cuda = _kernel()

    def reset_cache(self, batch_size: int, max_seq_len: int) -> None:
        self.attention.reset_cache(batch_size, max_seq_len)

    def __call__(self, x: torch.Tensor, start_pos: int, *, in_place: bool = False) -> torch.Tensor:
        """x [batch, steps, dim] at positions start_pos ..; returns the residual stream behind the layer.  in_place: x may be
        overwritten (a layer stack passing its own tensor from layer to layer); otherwise the caller's tensor is left alone."""
        start_pos = int(start_pos)
        stream = x.to(self.dtype).contiguous()
        if stream is x and not in_place:
            stream = x.clone()
        rows = stream.numel() // stream.size(-1)
        o = self.attention.o_proj
        if rows <= 4:
            # decode: normalisation inside the q / k / v launch, residual added in the output projection's store
            ctx = self.attention.context(stream, start_pos, input_norm=self.attn_norm)
            self._cuda.gguf_quant_gemm_accumulate_forward(ctx.contiguous(), o.tensor.blocks, int(o.tensor.row_elems), int(o.tensor.type_id), o._grid,
                                                          stream)
        else:
            stream += self.attention(self.attn_norm(stream), start_pos)
        return self.moe(stream, residual=stream, input_norm=self.ffn_norm)


class MiniMaxTransformer:
    """The layer stack (reference: architecture.py:417-472): token embedding from raw blocks, the blocks, the final
    normalisation and the vocabulary projection of the last position (or of all).  One GPU, so logits are whole rows."""

    def __init__(self, args: MiniMaxM2Args, embedding, layers: list[MiniMaxBlock], final_norm_weight: torch.Tensor, lm_head: QuantizedGGUFLinear,
                 *, device: torch.device, dtype: torch.dtype = torch.float16):
        self.args = args
        self.embedding = embedding
        self.layers = list(layers)
        self.final_norm = RMSNorm(final_norm_weight, args.norm_eps, out_dtype=dtype)
        self.lm_head = lm_head
        self.device = device
        self.dtype = dtype
        self._cuda = _kernel()

    def reset_cache(self, batch_size: int, max_seq_len: int) -> None:
        for layer in self.layers:
            layer.reset_cache(batch_size, max_seq_len)

    @torch.inference_mode()
    def forward(self, tokens: torch.Tensor, start_pos: int = 0, *, return_next_token: bool = False, keep_all_positions: bool = False):
        """tokens [batch, steps] (or [steps]) at positions start_pos ..; float32 logits [batch, 1 or steps, vocabulary], or the
        arg-max token ids when return_next_token is set."""
        ids = tokens.to(self.device)
        ids = ids.view(1, -1) if ids.dim() == 1 else ids
        hidden = self.embedding(ids).to(self.dtype)
        for layer in self.layers:
            hidden = layer(hidden, int(start_pos), in_place=True)                # `hidden` is this call's own tensor
        if not keep_all_positions:
            hidden = hidden[:, -1:, :]
        hidden = hidden.contiguous()
        head = self.lm_head.tensor
        if hidden.numel() // hidden.size(-1) <= 4 and int(head.row_start) == 0 and self._cuda is not None and hidden.is_cuda:
            # decode: the final normalisation inside the vocabulary projection's launch
            logits = self._cuda.gguf_quant_gemm_rmsnorm_forward(hidden, self.final_norm.weight, self.final_norm.eps, head.blocks, int(head.row_elems),
                                                                int(head.type_id), self.lm_head._grid, out_dtype=self.lm_head.out_dtype).float()
        else:
            logits = self.lm_head(self.final_norm(hidden)).float()
        if return_next_token:
            best = logits.argmax(dim=-1)
            return best if keep_all_positions else best[:, -1]
        return logits

    __call__ = forward
