"""Grouped-query causal attention over the paged cache (the Llama mixer).

Per token: q, k, v = h Wq^T, h Wk^T, h Wv^T (tiny_llm/ops/cuda/gemm.cu:86-100,
head-major columns gemm.cu:119-123); q and k rotated by the token's position
(rope.cu:46-54); k (rotated) and v written to the cache (gemm.cu:400-407);
scores q.k * hd^-0.5 against the request's cached keys with a causal mask, online
softmax, weighted sum of values (flash_attention.cu:374-405); output projection
with the residual add folded in (gemm.cu:171-190, arithmetic.cu:13).

Q, K and V weights are concatenated on load into one [(nq + 2 nkv) * hd, H]
matrix: row concatenation leaves every dot product as it was.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .norm import LazyNorm
from .base import (CacheSpec, LayerCache, Mixer, POSITION_ENCODINGS, WeightSpec, project_into_residual,
                   register_mixer)


class Attention(Mixer):
    graph_safe = True
    accepts_lazy_norm = True
    prepares_next_norm = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, position: dict = None, window: int = 0, scale: float = None,
                 max_position: int = 0):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        if self.num_kv_heads <= 0 or self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        # sizes a kernel refuses are refused here, when the model is built, not at its first step
        ops.check_attention_sizes(dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.num_heads * self.head_dim, f"{prefix}: num_heads * head_dim")
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        pos = dict(position or {"kind": "none"})
        kind = pos.pop("kind")
        self.position = POSITION_ENCODINGS.get(kind)(f"{prefix}.position", dtype, device, **pos)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    # ---------------------------------------------------------------- declarations
    def weights(self) -> List[WeightSpec]:
        p, H = self.prefix, self.hidden_size
        return [WeightSpec(f"{p}.q_proj.weight", (self.q_size, H)),
                WeightSpec(f"{p}.k_proj.weight", (self.kv_size, H)),
                WeightSpec(f"{p}.v_proj.weight", (self.kv_size, H)),
                WeightSpec(f"{p}.o_proj.weight", (H, self.q_size))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        self.w_qkv = torch.cat([tensors[f"{p}.q_proj.weight"], tensors[f"{p}.k_proj.weight"],
                                tensors[f"{p}.v_proj.weight"]], dim=0).contiguous()
        self.w_o = tensors[f"{p}.o_proj.weight"].contiguous()

    def cache_spec(self) -> CacheSpec:
        return CacheSpec.keys_and_values(self.num_kv_heads, self.head_dim, "window" if self.window else "full",
                                         self.window)

    # --------------------------------------------------------------------- compute
    def forward(self, h, ctx, cache: LayerCache, state, residual, next_norm=None):
        T = residual.shape[0]
        qkv = ops.scratch("qkv", (T, self.q_size + 2 * self.kv_size), self.dtype, residual.device)
        if isinstance(h, LazyNorm):
            h.linear(self.w_qkv, qkv)
        else:
            ops.linear(h, self.w_qkv, qkv)
        tables = self.position.rotary_tables()
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        pairing = getattr(self.position, "pairing", "half")     # an encoding that says nothing pairs (i, i + rot/2)
        attn = ops.scratch("attention_out", (T, self.q_size), self.dtype, residual.device)
        q = qkv[:, :self.q_size]
        flash = ops.flash_attention_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        # decode steps: rotation and cache write ride in the attention kernel
        fuse = flash and ctx.max_q_len == 1 and cache.write and rot == self.head_dim and pairing == "half"
        if not fuse:
            slots = ctx.slot_mappings[cache.group] if cache.write else None
            ops.rope_store(qkv, ctx.positions, cos, sin, slots, cache.k if cache.write else None,
                           cache.v if cache.write else None, self.num_heads, self.num_kv_heads, self.head_dim, rot,
                           pairing)
        self._attend(q, ctx, cache, attn, fused_rope=(cos, sin) if fuse else None)
        out, prepared = project_into_residual(attn, self.w_o, residual, next_norm)
        return out if next_norm is None else (out, prepared)

    def _attend(self, q, ctx, cache: LayerCache, attn, fused_rope=None, sink: bool = False):
        """attn <- attention of the step's query rows q [T, heads * head_dim] over the cache, by the kernel that
        takes this step's shape.  sink: one more term exp(0) in every softmax's denominator."""
        T, device = q.shape[0], q.device
        group = self.num_heads // self.num_kv_heads
        flash = ops.flash_attention_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        # the keys one row walks at most: a window bounds them whatever the context (the kernels begin at the
        # window's first key tile)
        span = min(ctx.max_seq_len, self.window + 63) if self.window else ctx.max_seq_len
        if flash and ctx.max_q_len > 1:
            # prompt portions: many query rows share each staged key tile
            waves = ops.prefill_tile_waves(T, self.num_heads, self.num_kv_heads)
            tiles = ctx.attention_tiles(waves * (16 // group))
            # a portion late in a long prompt: few query rows, many keys; the keys are shared out
            n_splits = ops.prefill_key_splits(T, span, self.num_heads, self.num_kv_heads, waves)
            scratch = None
            if n_splits > 1:
                scratch = ops.scratch("attention_partials", (n_splits * T * self.num_heads * (self.head_dim + 2),),
                                      torch.float32, device)
            ops.flash_prefill(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, waves,
                              n_splits, scratch, sink=sink)
        elif flash:
            # decoding: one token per request, its keys split over the waves of a workgroup (and over
            # workgroups when the context is long)
            # (no tile arrays when every request brings exactly one token: row i is request i)
            tiles = None if T == ctx.num_requests else ctx.attention_tiles(16 // group)
            n_splits, scratch = self._splits(span, T, device)
            ops.flash_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                                self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window,
                                n_splits, scratch, fused_rope=fused_rope, sink=sink)
        elif ops.attention_f32_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim) \
                and q.stride(0) % 4 == 0:
            # true float32 on the matrix cores; one fixed merge tree, so the same bits whatever the batch
            decode = ctx.max_q_len == 1 and T == ctx.num_requests
            tiles = None if decode else ctx.attention_tiles(16 // group)
            n_chunks = -(-ctx.max_seq_len // ops.F32_CHUNK_KEYS) if ctx.max_q_len == 1 else 1
            scratch = None
            if n_chunks > 1:
                scratch = ops.scratch("attention_partials", (n_chunks * T * self.num_heads * (self.head_dim + 2),),
                                      torch.float32, device)
            ops.attention_f32(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, n_chunks,
                              scratch, sink=sink)
        else:
            ops.paged_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.req_of_token,
                                ctx.positions, attn, self.num_heads, self.num_kv_heads, self.head_dim,
                                self.scale, self.window, sink=sink)
        return attn

    def _splits(self, span: int, T: int, device):
        """How many workgroups share one query tile's keys (`ops.decode_key_splits`; `span`: the most keys a
        row walks), and the scratch for their partial results."""
        n_splits = ops.decode_key_splits(T, span, self.num_kv_heads, self.head_dim)
        if n_splits == 1:
            return 1, None
        return n_splits, ops.scratch("attention_partials", (n_splits * T * self.num_heads * (self.head_dim + 2),),
                                     torch.float32, device)


class NormedAttention(Attention):
    """Grouped-query attention over the paged cache whose queries and keys are prepared in float32 between
    their product and the attention kernel, each step an option of its own:

        q, k = W_q h (+ b_q), W_k h (+ b_k)             `bias`
        v    = k as projected (`values="keys"`, no W_v), or W_v h (`values="projected"`)
        q, k rotated on the first rotary_dim dims of every head (`position`, either pairing)
        q, k divided by their root mean square over the head (`qk_norm="unit"`, no weight, `eps`)
        p_j  = exp(s_j) / (1 + sum exp(s_j))            `sink`: a term of score 0 that carries no value
        head n's output times sigmoid(W_g h)_n          `head_gate`: one number per token and head
        result = out_scale * W_o concat_heads(...)

    `window` and `scale` as in `Attention`.  `names`: the tensors' names below the prefix (q, k, v, g, o;
    a bias is its matrix's name plus `bias_suffix`).  One product reads h for [q | k | (v) | g] and leaves
    float32; the gate and `out_scale` are applied to the attention's result in float32 before it is
    rounded for the output product.  With `residual=None` the result is returned by itself in float32."""
    graph_safe = True
    accepts_lazy_norm = False
    prepares_next_norm = False

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: dict = None, window: int = 0, scale: float = None, bias: bool = False,
                 values: str = "projected", qk_norm: str = None, eps: float = 1e-6, sink: bool = False,
                 head_gate: bool = False, out_scale: float = 1.0, names: Dict[str, str] = None,
                 bias_suffix: str = ".bias", max_position: int = 0):
        super().__init__(prefix, dtype, device, hidden_size=hidden_size, num_heads=num_heads,
                         num_kv_heads=num_kv_heads, head_dim=head_dim, position=position, window=window, scale=scale)
        if values not in ("projected", "keys"):
            raise ValueError(f"{prefix}: values are 'projected' or 'keys', got {values!r}")
        if qk_norm not in (None, "unit"):
            raise ValueError(f"{prefix}: qk_norm is None or 'unit', got {qk_norm!r}")
        if self.head_dim % 2:
            raise ValueError(f"{prefix}: head_dim {self.head_dim} must be even")
        if float(out_scale) != 1.0 and not head_gate:
            raise ValueError(f"{prefix}: out_scale rides in the head gate's kernel; without a gate it must be 1")
        self.bias, self.values_are_keys, self.unit_norm = bool(bias), values == "keys", qk_norm == "unit"
        self.eps, self.sink, self.head_gate, self.out_scale = float(eps), bool(sink), bool(head_gate), float(out_scale)
        n = {k: k for k in ("q", "k", "v", "g", "o")}
        n.update(names or {})
        self.names = {k: f"{prefix}.{v}" for k, v in n.items()}
        self.bias_suffix = bias_suffix
        # columns of the product that reads h: q heads, k heads, (v heads,) then the gates at a multiple of 8
        self.v_off = self.q_size + self.kv_size if not self.values_are_keys else -1
        used = self.q_size + self.kv_size * (1 if self.values_are_keys else 2)
        self.g_off = -(-used // 8) * 8
        self.in_width = self.g_off + (-(-self.num_heads // 8) * 8 if self.head_gate else 0)
        self.w_in = self.b_in = None

    def weights(self) -> List[WeightSpec]:
        n, H = self.names, self.hidden_size
        out = [WeightSpec(n["q"], (self.q_size, H)), WeightSpec(n["k"], (self.kv_size, H))]
        if self.bias:
            out += [WeightSpec(n["q"] + self.bias_suffix, (self.q_size,), role="vector", init="zeros"),
                    WeightSpec(n["k"] + self.bias_suffix, (self.kv_size,), role="vector", init="zeros")]
        if not self.values_are_keys:
            out.append(WeightSpec(n["v"], (self.kv_size, H)))
        if self.head_gate:
            out.append(WeightSpec(n["g"], (self.num_heads, H)))
        out.append(WeightSpec(n["o"], (H, self.q_size)))
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        dev = tensors[n["q"]].device
        w = torch.zeros((self.in_width, self.hidden_size), dtype=self.dtype, device=dev)
        w[:self.q_size] = tensors[n["q"]]
        w[self.q_size:self.q_size + self.kv_size] = tensors[n["k"]]
        if not self.values_are_keys:
            w[self.v_off:self.v_off + self.kv_size] = tensors[n["v"]]
        if self.head_gate:
            w[self.g_off:self.g_off + self.num_heads] = tensors[n["g"]]
        self.w_in = w
        if self.bias:
            self.b_in = torch.cat([tensors[n["q"] + self.bias_suffix].to(torch.float32),
                                   tensors[n["k"] + self.bias_suffix].to(torch.float32)]).contiguous()
        self.w_o = tensors[n["o"]].contiguous()

    def forward(self, h, ctx, cache: LayerCache, state, residual):
        T, dev = h.shape[0], h.device
        p = ops.scratch("qk_product", (T, self.in_width), torch.float32, dev)
        ops.linear(h, self.w_in, p)
        tables = self.position.rotary_tables()
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        pairing = getattr(self.position, "pairing", "half")
        q = ops.scratch("q_prepared", (T, self.q_size), self.dtype, dev)
        write = cache.write
        ops.qk_prepare(p, self.b_in, ctx.positions, cos, sin, ctx.slot_mappings[cache.group] if write else None, q,
                       cache.k if write else None, cache.v if write else None, self.num_heads, self.num_kv_heads,
                       self.head_dim, rot, pairing, self.unit_norm, self.eps, self.values_are_keys, self.v_off)
        attn = ops.scratch("attention_out", (T, self.q_size), self.dtype, dev)
        self._attend(q, ctx, cache, attn, sink=self.sink)
        if self.head_gate:
            ops.head_gate(attn, p[:, self.g_off:self.g_off + self.num_heads], attn, self.num_heads, self.head_dim,
                          self.out_scale)
        if residual is None:
            return ops.linear(attn, self.w_o, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(attn, self.w_o, residual, residual)


register_mixer("attention", Attention)
register_mixer("normed_attention", NormedAttention)
