"""Prefill of one sequence of a W4A16 / Q8-KV transformer as a list of kernel dispatches.

The step on the other side of the KV cache from `decode_step.py`: all tokens of a prompt go
through every layer at once - RMSNorm + fused QKV projection (the prefill GEMM), RoPE on Q and K
(token-major in, head-major out, as llmopt_rotary_qk_f16_simd_h64 writes them), the Q8 pack of
every token's K and V into its pool slot (lib/serving_engine.ml:409-421 is where the reference
does this after a prefill), causal dense fp16 attention over the fresh K/V
(lib/metal_dispatch_attention.ml:6-102), output projection with the residual, the SwiGLU FFN -
and the LM-head argmax of the last token gives the first generated token.  Afterwards the pool
holds the prompt, and a `DecodeStep` over the same pool and slot table continues from there.

Reference entry points plus the extensions `decode_step.py` also uses - the two normalising
projection entries and, unless `reference_entries` is set, the rotation fused with the Q8 pack
(`llmopt_rotary_qk_pack_q8_batched` in place of the rotation and two cache packs: the same bytes
out); every entry is (kernel name, buffers, parameter block, grid, threadgroup).  V leaves the QKV
projection token-major [tokens, kv_heads * head_dim]: the attention entry takes it as it is
(token_first_value), and the cache pack reads it as ONE head of kv_heads * head_dim values, whose
64-wide groups are the same bytes and scales as the per-head groups of the head-major layout.
"""
from __future__ import annotations

import math
import struct

import numpy as np

from .decode_step import DecodeConfig, linear_grid, rope_rows, u32s
from .native import Buffer, Runtime


class PrefillStep:
    """Device buffers and the dispatch list that prefills `tokens` prompt tokens of one sequence
    into pool slots `slots[0 .. tokens)` (positions 0 .. tokens - 1)."""

    def __init__(self, runtime: Runtime, config: DecodeConfig, weights: dict, tokens: int, pool: Buffer,
                 slots: Buffer, device_weights: dict | None = None, reference_entries: bool = False):
        if tokens < 2:
            raise ValueError("a prefill has at least two tokens (one token is a decode step)")
        if config.head_dim not in (64, 128, 256, 512):
            raise ValueError("dense attention entries exist for head sizes 64, 128, 256 and 512")
        self.runtime, self.config, self.token_count = runtime, config, tokens
        self.reference_entries = reference_entries
        b = runtime.buffer_of_bytes
        c = config
        self.pool, self.slots = pool, slots
        self.tokens = b(np.zeros(tokens, dtype=np.int64))
        self.token_id = b(np.zeros(1, dtype=np.uint32))
        cos, sin = rope_rows(c, np.arange(tokens))
        self.cos, self.sin = b(cos), b(sin)
        self.device = device_weights if device_weights is not None else {
            "embedding": b(weights["embedding"]),
            "final_norm": b(weights["final_norm"]),
            "lm_head": tuple(b(a) for a in weights["lm_head"]),
            "layers": [{key: (tuple(b(a) for a in value) if isinstance(value, tuple) else b(value))
                        for key, value in layer.items()} for layer in weights["layers"]],
        }
        create = runtime.create_buffer
        h, qd, kvd = c.hidden, c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        self.work = {
            "x": [create(tokens * h * 2), create(tokens * h * 2)],
            "q": create(tokens * qd * 2), "k": create(tokens * kvd * 2), "v": create(tokens * kvd * 2),
            "q_rot": create(tokens * qd * 2), "k_rot": create(tokens * kvd * 2),
            "attention": create(tokens * qd * 2),
            "product": create(tokens * c.mlp * 2),
        }
        # the LM head reads the last token's row of the residual stream
        self.last_row = self.work["x"][0].view((tokens - 1) * h * 2, h * 2)
        self.dispatches = self._build()

    def _build(self) -> list[tuple]:
        c, t, w = self.config, self.token_count, self.work
        h, qd, kvd = c.hidden, c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        group = (256, 1, 1)
        rows_grid = lambda columns: (linear_grid(((t + 3) // 4) * columns), 1, 1)
        out: list[tuple] = []
        out.append(("llmopt_embedding_f16", [self.tokens, self.device["embedding"], w["x"][0]],
                    u32s(t, c.vocabulary, h), (((t * h + 255) // 256) * 256, 1, 1), group))
        pack = lambda offset, heads, width: u32s(t, offset, heads, width, 64, c.token_elements,
                                                 c.token_elements // 64, c.token_stride, t, 0)
        attention_params = struct.pack("<8IfIIIII", 1, c.q_heads, t, t, c.head_dim, 0, 0, 1,
                                       1.0 / math.sqrt(c.head_dim), c.kv_heads, 1, 0, 1, 0)
        for index, layer in enumerate(self.device["layers"]):
            x_in, x_mid = w["x"][0], w["x"][1]
            key_offset = index * c.layer_elements
            value_offset = key_offset + kvd
            out.append(("llmopt_rms_w4a16_qkv_linear_f16_g64",
                        [x_in, layer["attn_norm"], *layer["q"], *layer["k"], *layer["v"], w["q"], w["k"], w["v"]],
                        u32s(t, h, qd, kvd, kvd) + struct.pack("<f", c.epsilon), rows_grid(qd + 2 * kvd), group))
            if self.reference_entries:
                out.append(("llmopt_rotary_qk_f16_simd_h64",
                            [w["q"], w["k"], self.cos, self.sin, w["q_rot"], w["k_rot"]],
                            u32s(1, t, c.q_heads, c.kv_heads, c.head_dim, c.head_dim // 2, 1),
                            (((t * (c.q_heads + c.kv_heads) + 3) // 4) * 256, 1, 1), group))
                # K head-major [kv_heads, tokens, d]; V token-major = one head of kv_heads * d values
                out.append(("llmopt_cache_pack_attention_q8_simd", [w["k_rot"], self.slots, self.pool],
                            pack(key_offset, c.kv_heads, c.head_dim), (t * kvd // 64 * 32, 1, 1), group))
                out.append(("llmopt_cache_pack_attention_q8_simd", [w["v"], self.slots, self.pool],
                            pack(value_offset, 1, kvd), (t * kvd // 64 * 32, 1, 1), group))
            else:
                # rotation and every token's Q8 slot in one launch: the same bytes out, two launches fewer a layer
                out.append(("llmopt_rotary_qk_pack_q8_batched",
                            [w["q"], w["k"], self.cos, self.sin, w["q_rot"], w["k_rot"], w["v"], self.slots, self.pool],
                            u32s(1, t, c.q_heads, c.kv_heads, c.head_dim, c.head_dim // 2, 1) +
                            u32s(t, key_offset, value_offset, c.kv_heads, c.head_dim, 64, c.token_elements,
                                 c.token_elements // 64, c.token_stride, t, 0),
                            (((t * (c.q_heads + 2 * c.kv_heads) + 3) // 4) * 256, 1, 1), group))
            out.append((f"llmopt_attention_f16_simd_h{c.head_dim}",
                        [w["q_rot"], w["k_rot"], w["v"], w["q_rot"], w["attention"]], attention_params,
                        (t * c.q_heads, 1, 1), (64, 1, 1)))
            out.append(("llmopt_w4a16_linear_f16_g64_m4", [w["attention"], *layer["o"], x_in, x_mid],
                        u32s(t, h, qd, 1, h), rows_grid(h), group))
            ffn_params = u32s(t, c.mlp, h) + struct.pack("<f", c.epsilon)
            out.append(("llmopt_rms_w4a16_dual_swiglu_f16_g64",
                        [x_mid, layer["ffn_norm"], *layer["gate"], *layer["up"], w["product"]], ffn_params,
                        rows_grid(c.mlp), group))
            out.append(("llmopt_w4a16_down_add_f16_g64_m4", [w["product"], *layer["down"], x_mid, x_in], ffn_params,
                        rows_grid(h), group))
        out.append(("llmopt_w4a16_lm_head_argmax_f16",
                    [self.last_row, self.device["final_norm"], *self.device["lm_head"], self.token_id],
                    u32s(1, c.vocabulary, h) + struct.pack("<f", c.epsilon), (256, 1, 1), group))
        return out

    def record(self, batch) -> None:
        for name, buffers, parameters, grid, group in self.dispatches:
            batch.dispatch(name, buffers, parameters, grid=grid, group=group)

    def run(self, tokens) -> int:
        """Prefills the prompt; returns the first generated token id."""
        tokens = np.asarray(tokens, dtype=np.int64)
        if tokens.shape != (self.token_count,):
            raise ValueError(f"this step was built for {self.token_count} tokens")
        self.tokens.write(tokens)
        batch = self.runtime.begin_batch()
        self.record(batch)
        batch.commit()
        return int(self.token_id.numpy(np.uint32, (1,))[0])

    def flops(self) -> float:
        """Algorithmic flops of one prefill: the projections (2 M N K each), causal attention
        (4 h d L(L+1)/2 per layer) and the LM head of the last token."""
        c, t = self.config, self.token_count
        h, qd, kvd = c.hidden, c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        layer = 2.0 * t * h * (qd + 2 * kvd) + 2.0 * t * qd * h + 3 * 2.0 * t * h * c.mlp
        layer += 4.0 * c.q_heads * c.head_dim * t * (t + 1) / 2
        return c.layers * layer + 2.0 * h * c.vocabulary
