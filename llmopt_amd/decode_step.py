"""One decode step of a W4A16 / Q8-KV transformer as a list of kernel dispatches.

The host-side counterpart of what the reference's schedule executor encodes
for a decode step (lib/metal_schedule_executor.ml via lib/metal_dispatch_*.ml):
per layer RMSNorm, fused QKV projection, RoPE on Q and K, Q8 pack of the new
K/V, paged Q8 attention, output projection with the residual as addend, and
the three-launch SwiGLU FFN; then the LM-head argmax.  Every entry is
(kernel name, buffers, parameter block, grid, threadgroup) in the reference's
buffer order, ready for Batch.dispatch or a Prebaked plan.

Sequences of a batch have their own context lengths and slot tables, which the
batched attention / pack entry points take as two extra buffers.

A step list is built once.  What changes from token to token - the input
tokens, each sequence's context length, the slot of the new token, the rotary
rows of the new position - lives in device buffers the kernels read, so the
same list (or a Prebaked plan frozen from it) serves every step: `advance`
rewrites those buffers after a step.
"""
from __future__ import annotations

import functools
import math
import struct
from dataclasses import dataclass

import numpy as np

from .native import Buffer, Runtime


# Up to this many sequences a step takes the fused layer of three launches; above it every workgroup
# re-reading and re-decoding its weights per sequence costs more than the launches saved, and the step takes
# five launches a layer (the fused QKV launch in front of the reference's entries).  Measured at 2048 tokens
# of context, ms per step as three / five / six launches a layer: batch 1 0.703 / - / 0.794, 6 0.814 / 0.914 /
# -, 8 0.828 / 0.926 / 1.048, 10 0.908 / 0.966 / -, 12 1.014 / 0.988 / 1.077, 14 1.040 / 1.023 / -,
# 16 1.050 / 1.048 / 1.141, 20 1.161 / 1.168 / 1.263, 24 1.292 / 1.187 / 1.280, 32 1.361 / 1.232 / 1.324,
# 64 - / 1.705 / 1.890, 128 - / 2.722 / 2.759.
FUSED_MAX_BATCH = 10
# The attention launch multiplies its heads into the output projection where it can (three launches a
# layer instead of four: batch 1 0.742 against 0.771 ms, 8 0.856 / 0.907, 16 1.052 / 1.096, 32 1.364 / 1.379).
PROJECTING_ATTENTION = True
# Columns of the intermediate per workgroup of the fused FFN launch (and per partial sum it leaves): 32 where that
# stays within the 48 partial sums a reader takes, else 64.
FFN_SLICE = 32


def u32s(*values) -> bytes:
    """Metal_parameters.u32s (lib/metal_parameters.ml:14-22)."""
    return struct.pack("<%dI" % len(values), *values)


def linear_grid(columns: int) -> int:
    """linear_f16_grid (lib/metal_dispatch_common.ml:64-70)."""
    return ((columns + 7) // 8) * 8 * 32


@functools.lru_cache(maxsize=None)
def _kv_layout(layers: int, kv_heads: int, head_dim: int):
    from . import ops
    return ops.kv_layout([(kv_heads, head_dim)] * layers)


@dataclass(frozen=True)
class DecodeConfig:
    hidden: int = 576
    q_heads: int = 9
    kv_heads: int = 3
    head_dim: int = 64
    mlp: int = 1536
    layers: int = 30
    vocabulary: int = 49152
    epsilon: float = 1e-5
    rope_theta: float = 10000.0

    @property
    def kv_layout(self):
        """Kv_cache.Layout of this model's attention layers (lib/kv_cache.ml:126-166), from the
        library's llmopt_op_kv_layout."""
        return _kv_layout(self.layers, self.kv_heads, self.head_dim)

    @property
    def layer_elements(self) -> int:
        """Keys plus values of one layer in a token's slot (layers are uniform here: the key offset
        of layer i is i * layer_elements, its values follow its keys)."""
        key_offset, value_offset, segment, _ = self.kv_layout.regions[0]
        return 2 * segment

    @property
    def token_elements(self) -> int:
        return self.kv_layout.token_elements

    @property
    def token_stride(self) -> int:
        """Bytes per token: int8 values + one f16 scale per 64."""
        return self.kv_layout.bytes_per_token


def rope_rows(config: DecodeConfig, positions) -> tuple[np.ndarray, np.ndarray]:
    """cos / sin rows for the given positions, duplicated into both halves
    (Serving_rope_table.create, lib/serving_rope_table.ml:156-172): the angle is
    f32(inv_freq * f32(position)), cos/sin in f64 -> f32 -> f16."""
    d = config.head_dim
    inv_freq = (config.rope_theta ** (-np.arange(0, d, 2, dtype=np.float64) / d)).astype(np.float32)
    angle = (inv_freq[None, :] * np.asarray(positions, dtype=np.float32)[:, None]).astype(np.float32)
    cos = np.cos(angle.astype(np.float64)).astype(np.float32).astype(np.float16)
    sin = np.sin(angle.astype(np.float64)).astype(np.float32).astype(np.float16)
    return np.concatenate([cos, cos], axis=1), np.concatenate([sin, sin], axis=1)


def random_w4(rng, n: int, k: int):
    packed = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    scale = rng.uniform(0.005, 0.02, size=(n, k // 64)).astype(np.float16)
    return packed, scale


def random_weights(config: DecodeConfig, rng) -> dict:
    """Random-init weights in the reference's formats (host arrays)."""
    h, kv = config.hidden, config.kv_heads * config.head_dim
    layers = []
    for _ in range(config.layers):
        layers.append({
            "attn_norm": rng.uniform(0.5, 1.5, h).astype(np.float16),
            "q": random_w4(rng, config.q_heads * config.head_dim, h),
            "k": random_w4(rng, kv, h),
            "v": random_w4(rng, kv, h),
            "o": random_w4(rng, h, config.q_heads * config.head_dim),
            "ffn_norm": rng.uniform(0.5, 1.5, h).astype(np.float16),
            "gate": random_w4(rng, config.mlp, h),
            "up": random_w4(rng, config.mlp, h),
            "down": random_w4(rng, h, config.mlp),
        })
    return {
        "embedding": (rng.standard_normal((config.vocabulary, h)) * 0.5).astype(np.float16),
        "layers": layers,
        "final_norm": rng.uniform(0.5, 1.5, h).astype(np.float16),
        "lm_head": random_w4(rng, config.vocabulary, h),
    }


class DecodeStep:
    """Device buffers and the dispatch list of one decode step for `batch` sequences."""

    def __init__(self, runtime: Runtime, config: DecodeConfig, weights: dict, batch: int, pool: Buffer,
                 slots: Buffer, slot_offsets, past_lengths, new_slots, positions, max_context=None,
                 slots_host=None, reference_entries: bool = False, fused: bool | None = None,
                 projecting: bool | None = None, fused_qkv: bool | None = None):
        """max_context: the longest context any later step will have (sizes the attention launch;
        default: the longest now).  slots_host: the host copy of the slot table, with room behind
        every sequence's slots for the tokens `advance` will add.  reference_entries (batch 1):
        rotation, cache pack and attention as the reference's own three kernels
        (llmopt_rotary_qk_f16_simd_h64, llmopt_cache_pack_attention_q8_pair_simd,
        llmopt_attention_q8_paged_simd_h64_gqa3) instead of the batched extension entries.
        fused (default: whenever the shapes allow and reference_entries is off): norm + QKV + rotation
        + cache pack as one launch, attention, output projection, and the SwiGLU FFN as one that leaves
        partial sums for the next layer's first launch - four launches a layer instead of six; three
        where the attention launch can multiply its heads into the output projection itself
        (`self.projecting`: contexts of 64 tokens and more, hidden <= 1024, at most 32 query heads).
        fused_qkv (a step that is not `fused`; default: whenever the shapes allow): the first of those launches
        in front of the reference's entries for the rest of the layer - five launches a layer, which is what
        larger batches take (measured against six: 1.188 / 1.280 ms at batch 24, 1.232 / 1.324 at 32,
        1.705 / 1.890 at 64, 2.722 / 2.759 at 128)."""
        self.runtime, self.config, self.batch = runtime, config, batch
        self.reference_entries = reference_entries
        if reference_entries and batch != 1:
            raise ValueError("the reference's paged attention entries share one slot table: batch 1")
        # (slices of 32 while their workgroups fit the device's 256 CUs once; measured at the 30-layer model:
        # batch 1 0.709 against 0.742 ms, 4 0.762 / 0.793, 8 0.873 / 0.856, 16 1.079 / 1.050)
        self.ffn_slice = FFN_SLICE if config.mlp % FFN_SLICE == 0 and config.mlp // FFN_SLICE <= 48 and \
            config.hidden <= 1024 and batch * (config.mlp // FFN_SLICE) <= 256 else 64
        can_fuse = (config.head_dim == 64 and config.hidden % 64 == 0 and config.hidden <= 1472 and
                    config.mlp % 64 == 0 and config.mlp // 64 <= 32)
        if fused and (reference_entries or not can_fuse):
            raise ValueError("the fused launches take heads of 64, hidden <= 1472 and mlp <= 2048")
        self.fused = can_fuse and not reference_entries and batch <= FUSED_MAX_BATCH if fused is None else fused
        can_fuse_qkv = (not self.fused and not reference_entries and config.head_dim == 64 and config.hidden % 64 == 0 and
                        config.hidden <= 2048)
        if fused_qkv and not can_fuse_qkv:
            raise ValueError("the fused QKV launch takes a step that is not fused, heads of 64 and hidden <= 2048")
        self.fused_qkv = can_fuse_qkv if fused_qkv is None else fused_qkv
        self.max_past = int(max(past_lengths)) if max_context is None else int(max_context)
        can_project = bool(self.fused and self.max_past >= 64 and config.hidden <= 1024 and config.q_heads <= 32)
        if projecting and not can_project:
            raise ValueError("the projecting attention takes a fused step, contexts of 64 tokens and more, "
                             "hidden <= 1024 and at most 32 query heads")
        self.projecting = can_project and PROJECTING_ATTENTION if projecting is None else projecting
        self.host_lengths = np.asarray(past_lengths, dtype=np.uint32).copy()
        self.host_offsets = np.asarray(slot_offsets, dtype=np.uint32).copy()
        self.host_positions = np.asarray(positions, dtype=np.int64).copy()
        self.slots_host = None if slots_host is None else np.asarray(slots_host, dtype=np.uint32)
        b = runtime.buffer_of_bytes
        c = config
        h = c.hidden
        self.pool, self.slots = pool, slots
        self.tokens = b(np.zeros(batch, dtype=np.int64))
        self.token_ids = b(np.zeros(batch, dtype=np.uint32))
        self.past_lengths = b(np.asarray(past_lengths, dtype=np.uint32))
        self.slot_offsets = b(np.asarray(slot_offsets, dtype=np.uint32))
        self.new_slots = b(np.asarray(new_slots, dtype=np.uint32))
        cos, sin = rope_rows(c, positions)
        # cosine rows, then sine rows, in one buffer (the fused launch takes them as one)
        self.trig = b(np.concatenate([cos, sin]))
        self.cos = self.trig.view(0, cos.nbytes)
        self.sin = self.trig.view(cos.nbytes, sin.nbytes)
        self.device = {
            "embedding": b(weights["embedding"]),
            "final_norm": b(weights["final_norm"]),
            "lm_head": tuple(b(a) for a in weights["lm_head"]),
            "layers": [{key: (tuple(b(a) for a in value) if isinstance(value, tuple) else b(value))
                        for key, value in layer.items()} for layer in weights["layers"]],
        }
        create = runtime.create_buffer
        q_bytes, kv_bytes = batch * c.q_heads * c.head_dim * 2, batch * c.kv_heads * c.head_dim * 2
        self.work = {
            "x": [create(batch * h * 2), create(batch * h * 2)],
            "q": create(q_bytes), "k": create(kv_bytes), "v": create(kv_bytes),
            "q_rot": create(q_bytes), "k_rot": create(kv_bytes),
            "attention": create(q_bytes),
            "product": create(batch * c.mlp * 2),
        }
        if self.fused or self.fused_qkv:
            self.work["stream"] = create(batch * h * 2)
        if self.fused:
            self.work["partials"] = create((c.mlp // self.ffn_slice) * batch * h * 4)
        if self.projecting:
            self.work["head_partials"] = create(c.q_heads * batch * h * 4)
        self.dispatches = self._build()

    def _linear_entry(self, columns_of_one_row: int):
        """Kernel name suffix and grid of the reference's m = 1 / m > 1 choice
        (lib/metal_dispatch_linear.ml:349-395, 938-982)."""
        m = self.batch
        if m == 1:
            return "", (linear_grid(columns_of_one_row), 1, 1)
        return "_m4", (linear_grid(((m + 3) // 4) * columns_of_one_row), 1, 1)

    def _build(self) -> list[tuple]:
        c, m, w = self.config, self.batch, self.work
        h, qd, kvd = c.hidden, c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        group = (256, 1, 1)
        out: list[tuple] = []
        count = m * h
        out.append(("llmopt_embedding_f16", [self.tokens, self.device["embedding"], w["x"][0]],
                    u32s(m, c.vocabulary, h), (((count + 255) // 256) * 256, 1, 1), group))
        for index, layer in enumerate(self.device["layers"]):
            x_in, x_mid = w["x"][0], w["x"][1]
            key_offset = index * c.layer_elements
            value_offset = key_offset + kvd
            if self.fused:
                out += self._fused_layer(index, layer, key_offset, value_offset)
                continue
            if self.fused_qkv:
                # norm + QKV + rotation + cache pack as one launch (no pending sums: the stream is whole; the
                # copy of it that the launch writes is not read), the rest as the reference's entries
                out.append(("llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64",
                            [x_in, x_in, w["stream"], layer["attn_norm"], *layer["q"], *layer["k"], *layer["v"],
                             self.trig, w["q_rot"], w["k_rot"], w["v"], self.new_slots, self.pool],
                            u32s(m, h, qd, kvd, kvd) + struct.pack("<f", c.epsilon) +
                            u32s(0, key_offset, value_offset, c.token_elements, c.token_stride),
                            (((qd + 2 * kvd) // 64) * 256, m, 1), group))
                out.append(self._batched_attention(key_offset, value_offset))
                suffix, grid = self._linear_entry(h)
                out.append(("llmopt_w4a16_linear_f16_g64" + suffix,
                            [w["attention"], *layer["o"], x_in, x_mid], u32s(m, h, qd, 1, h), grid, group))
                ffn_params = u32s(m, c.mlp, h) + struct.pack("<f", c.epsilon)
                suffix, grid = self._linear_entry(c.mlp)
                out.append(("llmopt_rms_w4a16_dual_swiglu_f16_g64",
                            [x_mid, layer["ffn_norm"], *layer["gate"], *layer["up"], w["product"]], ffn_params, grid,
                            group))
                suffix, grid = self._linear_entry(h)
                out.append(("llmopt_w4a16_down_add_f16_g64" + suffix,
                            [w["product"], *layer["down"], x_mid, x_in], ffn_params, grid, group))
                continue
            # each RMSNorm rides in the projection launch that reads it
            suffix, grid = self._linear_entry(qd + 2 * kvd)
            out.append(("llmopt_rms_w4a16_qkv_linear_f16_g64",
                        [x_in, layer["attn_norm"], *layer["q"], *layer["k"], *layer["v"], w["q"], w["k"], w["v"]],
                        u32s(m, h, qd, kvd, kvd) + struct.pack("<f", c.epsilon), grid, group))
            if self.reference_entries:
                out += self._reference_attention(key_offset, value_offset)
            else:
                # rotation and the new token's Q8 slot in one launch (the step is bound by its launches)
                out.append(("llmopt_rotary_qk_pack_q8_batched",
                            [w["q"], w["k"], self.cos, self.sin, w["q_rot"], w["k_rot"], w["v"], self.new_slots,
                             self.pool],
                            u32s(m, 1, c.q_heads, c.kv_heads, c.head_dim, c.head_dim // 2, m) +
                            u32s(m, key_offset, value_offset, c.kv_heads, c.head_dim, 64, c.token_elements,
                                 c.token_elements // 64, c.token_stride, m, 0),
                            (((m * (c.q_heads + 2 * c.kv_heads) + 3) // 4) * 256, 1, 1), group))
                out.append(self._batched_attention(key_offset, value_offset))
            suffix, grid = self._linear_entry(h)
            out.append(("llmopt_w4a16_linear_f16_g64" + suffix,
                        [w["attention"], *layer["o"], x_in, x_mid], u32s(m, h, qd, 1, h), grid, group))
            ffn_params = u32s(m, c.mlp, h) + struct.pack("<f", c.epsilon)
            suffix, grid = self._linear_entry(c.mlp)
            out.append(("llmopt_rms_w4a16_dual_swiglu_f16_g64",
                        [x_mid, layer["ffn_norm"], *layer["gate"], *layer["up"], w["product"]], ffn_params, grid,
                        group))
            suffix, grid = self._linear_entry(h)
            out.append(("llmopt_w4a16_down_add_f16_g64" + suffix,
                        [w["product"], *layer["down"], x_mid, x_in], ffn_params, grid, group))
        out.append(("llmopt_w4a16_lm_head_argmax_f16",
                    [w["x"][0], self.device["final_norm"], *self.device["lm_head"], self.token_ids],
                    u32s(m, c.vocabulary, h) + struct.pack("<f", c.epsilon), (m * 256, 1, 1), group))
        return out

    def _batched_attention(self, key_offset: int, value_offset: int, projection=None) -> tuple:
        """projection: the output projection's (weights, scales) for the entry that leaves every head's
        share of it as float32 partial sums instead of the attention rows."""
        c, m, w = self.config, self.batch, self.work
        attention_params = struct.pack(
            "<12IfIII", m, c.q_heads, c.kv_heads, 0, c.head_dim, 0, 0, c.token_elements, key_offset,
            value_offset, 64, c.token_stride, 1.0 / math.sqrt(c.head_dim), 1, 0, 0)
        attention_params += struct.pack("<I", self.max_past)
        grid = (((m * c.q_heads + 7) // 8) * 256, 1, 1)
        if projection is not None:
            return ("llmopt_attention_q8_paged_batched_w4a16_partial_g64",
                    [w["q_rot"], w["k_rot"], w["v"], self.pool, self.slots, self.slots, w["head_partials"],
                     self.past_lengths, self.slot_offsets, *projection],
                    attention_params + struct.pack("<I", c.hidden), grid, (256, 1, 1))
        return ("llmopt_attention_q8_paged_batched",
                [w["q_rot"], w["k_rot"], w["v"], self.pool, self.slots, self.slots, w["attention"],
                 self.past_lengths, self.slot_offsets],
                attention_params, grid, (256, 1, 1))

    def _fused_layer(self, index: int, layer: dict, key_offset: int, value_offset: int) -> list[tuple]:
        """Four launches: the residual stream enters as the previous layer's `x_mid` plus the partial
        sums its FFN launch left (the first layer: the embedding rows, no sums); the last layer's FFN
        runs as the two reference entries, so that the LM head finds a whole stream."""
        c, m, w = self.config, self.batch, self.work
        h, qd, kvd = c.hidden, c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        group = (256, 1, 1)
        first, last = index == 0, index == c.layers - 1
        slices = c.mlp // self.ffn_slice
        stream_in = w["x"][0] if first else w["x"][1]
        out = [("llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64",
                [stream_in, w["partials"], w["stream"], layer["attn_norm"], *layer["q"], *layer["k"], *layer["v"],
                 self.trig, w["q_rot"], w["k_rot"], w["v"], self.new_slots, self.pool],
                u32s(m, h, qd, kvd, kvd) + struct.pack("<f", c.epsilon) +
                u32s(0 if first else slices, key_offset, value_offset, c.token_elements, c.token_stride),
                (((qd + 2 * kvd) // 64) * 256, m, 1), group)]
        ffn_params = u32s(m, c.mlp, h) + struct.pack("<f", c.epsilon)
        if self.projecting and not last:
            # three launches: the attention leaves each head's share of the output projection, the
            # FFN launch adds them to the stream on its way in
            out.append(self._batched_attention(key_offset, value_offset, projection=layer["o"]))
            out.append(("llmopt_sum_rms_w4a16_swiglu_down_partial_f16_g64",
                        [w["stream"], w["head_partials"], w["x"][1], layer["ffn_norm"], *layer["gate"], *layer["up"],
                         *layer["down"], w["partials"]],
                        ffn_params + u32s(c.q_heads, self.ffn_slice), (slices * 256, m, 1), group))
            return out
        out.append(self._batched_attention(key_offset, value_offset))
        suffix, grid = self._linear_entry(h)
        out.append(("llmopt_w4a16_linear_f16_g64" + suffix,
                    [w["attention"], *layer["o"], w["stream"], w["x"][1]], u32s(m, h, qd, 1, h), grid, group))
        if not last:
            out.append(("llmopt_rms_w4a16_swiglu_down_partial_f16_g64",
                        [w["x"][1], layer["ffn_norm"], *layer["gate"], *layer["up"], *layer["down"], w["partials"]],
                        ffn_params + u32s(self.ffn_slice), (slices * 256, m, 1), group))
            return out
        suffix, grid = self._linear_entry(c.mlp)
        out.append(("llmopt_rms_w4a16_dual_swiglu_f16_g64",
                    [w["x"][1], layer["ffn_norm"], *layer["gate"], *layer["up"], w["product"]], ffn_params, grid,
                    group))
        suffix, grid = self._linear_entry(h)
        out.append(("llmopt_w4a16_down_add_f16_g64" + suffix,
                    [w["product"], *layer["down"], w["x"][1], w["x"][0]], ffn_params, grid, group))
        return out

    def _reference_attention(self, key_offset: int, value_offset: int) -> list[tuple]:
        """One sequence through the reference's own kernels: RotaryQKParams (lib/metal_parameters.ml),
        AttentionCachePairParams and Q8PagedAttentionParams (lib/metal_cache_source.ml:22-34,352-369).
        The context length at parameter byte 12 is what a Prebaked plan patches per step."""
        c, w = self.config, self.work
        group = (256, 1, 1)
        rows = c.q_heads + 2 * c.kv_heads
        attention_params = struct.pack(
            "<12IfIII", 1, c.q_heads, c.kv_heads, int(self.host_lengths[0]), c.head_dim, 0, 0, c.token_elements,
            key_offset, value_offset, 64, c.token_stride, 1.0 / math.sqrt(c.head_dim), 1, 0, 0)
        name = "llmopt_attention_q8_paged_simd_h64_gqa3" if (c.head_dim, c.q_heads // c.kv_heads) == (64, 3) \
            else "llmopt_attention_q8_paged_simd_generic"
        return [
            ("llmopt_rotary_qk_f16_simd_h64", [w["q"], w["k"], self.cos, self.sin, w["q_rot"], w["k_rot"]],
             u32s(1, 1, c.q_heads, c.kv_heads, c.head_dim, c.head_dim // 2, 1), (((rows + 3) // 4) * 256, 1, 1), group),
            ("llmopt_cache_pack_attention_q8_pair_simd", [w["k_rot"], w["v"], self.new_slots, self.pool],
             u32s(1, key_offset, value_offset, c.kv_heads, c.head_dim, 64, c.token_elements, c.token_elements // 64,
                  c.token_stride, 1, 0), (c.kv_heads * (c.head_dim // 64) * 64, 1, 1), (64, 1, 1)),
            (name,
             [w["q_rot"], w["k_rot"], w["v"], self.pool, self.slots, self.slots, w["attention"]],
             attention_params, (((c.q_heads + 7) // 8) * 256, 1, 1), group),
        ]

    def set_reference_past(self, past_tokens: int) -> None:
        """Host-side patch of the context length (parameter byte 12) for eager runs of a reference_entries list."""
        patched = []
        for name, buffers, parameters, grid, group in self.dispatches:
            if name.startswith("llmopt_attention_q8_paged_simd"):
                parameters = parameters[:12] + struct.pack("<I", past_tokens) + parameters[16:]
            patched.append((name, buffers, parameters, grid, group))
        self.dispatches = patched

    def advance(self) -> None:
        """After a step: every sequence is one token longer.  Rewrites the device buffers the next
        step reads - context lengths, the new token's slot (the next entry of the sequence's slot
        table) and the rotary rows of the next position."""
        if self.slots_host is None:
            raise ValueError("advance needs the host copy of the slot table")
        self.host_lengths += 1
        self.host_positions += 1
        if int(self.host_lengths.max()) > self.max_past:
            raise ValueError("context grew beyond max_context")
        self.past_lengths.write(self.host_lengths)
        self.new_slots.write(self.slots_host[self.host_offsets + self.host_lengths])
        cos, sin = rope_rows(self.config, self.host_positions)
        self.cos.write(cos)
        self.sin.write(sin)
        if self.reference_entries:
            self.set_reference_past(int(self.host_lengths[0]))

    def record(self, batch) -> None:
        for name, buffers, parameters, grid, group in self.dispatches:
            batch.dispatch(name, buffers, parameters, grid=grid, group=group)

    def run(self, tokens) -> np.ndarray:
        """One eager step: returns the next token id of every sequence."""
        self.tokens.write(np.asarray(tokens, dtype=np.int64))
        batch = self.runtime.begin_batch()
        self.record(batch)
        batch.commit()
        return self.token_ids.numpy(np.uint32, (self.batch,))

    def weight_bytes(self) -> int:
        """Algorithmic weight bytes one step streams (packed weights + scales, the LM head included)."""
        c = self.config
        h, qd, kvd = c.hidden, c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        w4 = lambda n, k: n * k // 2 + 2 * n * (k // 64)
        layer = w4(qd, h) + 2 * w4(kvd, h) + w4(h, qd) + 2 * w4(c.mlp, h) + w4(h, c.mlp)
        return c.layers * layer + w4(c.vocabulary, h)

    def kv_bytes(self) -> int:
        """Algorithmic KV-cache bytes one step reads: every past token's whole pool slot."""
        total = int(self.past_lengths.numpy(np.uint32).sum())
        return total * self.config.token_stride
