"""Whole decode steps and prompt prefills composed from the CPU oracle (test infrastructure only).

The chains restate what the reference's schedule executor encodes per layer
(lib/metal_schedule_executor.ml:38-431 through lib/metal_dispatch_linear.ml:252-455,938-982 and
lib/metal_dispatch_attention.ml:104-217): RMSNorm, the Q / K / V projections, rotate-half position
encoding, the Q8 pack of the new K / V, paged Q8 (decode) or dense causal (prefill) attention, the
output projection with the residual, the SwiGLU FFN; then the final norm and the LM head's logits.
Every kernel boundary is rounded to half, as the kernels store it.  Only tests, the smoke check
and bench.py's checkers import this.

`config` is any object with hidden, q_heads, kv_heads, head_dim, mlp, epsilon, rope_theta,
layer_elements, token_elements and token_stride.
"""
from __future__ import annotations

import math

import numpy as np

import oracle
from oracle import CacheParams, PagedParams


def f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


def rope_rows(config, positions):
    """cos / sin rows of the given positions, duplicated into both halves
    (Serving_rope_table.create, lib/serving_rope_table.ml:156-172): the angle is
    f32(inv_freq * f32(position)), cos / sin in f64 -> f32 -> f16 (round to nearest even)."""
    d = config.head_dim
    inv_freq = (config.rope_theta ** (-np.arange(0, d, 2, dtype=np.float64) / d)).astype(np.float32)
    angle = (inv_freq[None, :] * np.asarray(positions, dtype=np.float32)[:, None]).astype(np.float32)
    cos = np.cos(angle.astype(np.float64)).astype(np.float32).astype(np.float16)
    sin = np.sin(angle.astype(np.float64)).astype(np.float32).astype(np.float16)
    return np.concatenate([cos, cos], axis=1), np.concatenate([sin, sin], axis=1)


def _cache_params(c, items, offset):
    return CacheParams(items=items, segment_offset=offset, heads=c.kv_heads, head_dim=c.head_dim, group_size=64,
                       token_elements=c.token_elements, token_groups=c.token_elements // 64,
                       token_stride=c.token_stride, source_items=items, source_offset=0)


def _ffn(c, layer, x_mid):
    n2 = f16(oracle.rms_norm(x_mid, layer["ffn_norm"], c.epsilon))
    product = f16(oracle.silu_mul(oracle.w4a16_linear(n2, *layer["gate"], None),
                                  oracle.w4a16_linear(n2, *layer["up"], None)))
    return f16(oracle.add(oracle.w4a16_linear(product, *layer["down"], None), x_mid.astype(np.float32)))


def decode_chain(config, weights, pool, slots, offsets, lengths, new_slots, positions, tokens):
    """One decode step of every sequence of a batch: the residual stream after the last layer
    [batch, hidden], the logits [batch, vocabulary] and the pool with the new tokens' K / V."""
    c = config
    pool = pool.copy()
    cos, sin = rope_rows(c, positions)
    hidden_out, logits_out = [], []
    for b, token in enumerate(tokens):
        x = weights["embedding"][token][None, :]
        seq_slots = slots[offsets[b]:offsets[b] + lengths[b]]
        for index, layer in enumerate(weights["layers"]):
            key_offset = index * c.layer_elements
            value_offset = key_offset + c.kv_heads * c.head_dim
            n1 = f16(oracle.rms_norm(x, layer["attn_norm"], c.epsilon))
            q = f16(oracle.w4a16_linear(n1, *layer["q"], None)).reshape(1, c.q_heads, c.head_dim)
            k = f16(oracle.w4a16_linear(n1, *layer["k"], None)).reshape(1, c.kv_heads, c.head_dim)
            v = f16(oracle.w4a16_linear(n1, *layer["v"], None)).reshape(1, c.kv_heads, c.head_dim)
            q_rot = f16(oracle.rotary_h(q, cos[b:b + 1], sin[b:b + 1]))   # [heads, 1, d]
            k_rot = f16(oracle.rotary_h(k, cos[b:b + 1], sin[b:b + 1]))
            v_heads = v.transpose(1, 0, 2).copy()
            for source, offset in ((k_rot, key_offset), (v_heads, value_offset)):
                oracle.q8_pack(source, np.array([new_slots[b]], dtype=np.uint32), pool, _cache_params(c, 1, offset))
            params = PagedParams(batches=1, query_heads=c.q_heads, kv_heads=c.kv_heads, past_length=lengths[b],
                                 head_dim=c.head_dim, mask_batches=0, mask_heads=0,
                                 token_elements=c.token_elements, key_offset=key_offset,
                                 value_offset=value_offset, group_size=64, token_stride=c.token_stride,
                                 scale=1.0 / math.sqrt(c.head_dim), query_length=1, mask_dtype=0, window=0)
            attention = f16(oracle.paged_attention_q8(q_rot[None], k_rot[None], v_heads[None], pool, seq_slots,
                                                      None, params)).reshape(1, -1)
            x_mid = f16(oracle.add(oracle.w4a16_linear(attention, *layer["o"], None), x.astype(np.float32)))
            x = _ffn(c, layer, x_mid)
        hidden_out.append(x[0])
        final = oracle.rms_norm(x, weights["final_norm"], c.epsilon)
        logits_out.append(oracle.w4a16_linear(final, *weights["lm_head"], None)[0])
    return np.stack(hidden_out), np.stack(logits_out), pool


def prefill_chain(config, weights, tokens, slots, pool):
    """A whole prompt at once: the residual stream [tokens, hidden], the last token's logits and
    the pool with every prompt token's K / V in its slot."""
    c = config
    t = len(tokens)
    pool = pool.copy()
    cos, sin = rope_rows(c, np.arange(t))
    x = weights["embedding"][np.asarray(tokens)]
    causal = np.tril(np.ones((t, t), dtype=np.float32))[None, None]
    for index, layer in enumerate(weights["layers"]):
        key_offset = index * c.layer_elements
        value_offset = key_offset + c.kv_heads * c.head_dim
        n1 = f16(oracle.rms_norm(x, layer["attn_norm"], c.epsilon))
        q = f16(oracle.w4a16_linear(n1, *layer["q"], None)).reshape(t, c.q_heads, c.head_dim)
        k = f16(oracle.w4a16_linear(n1, *layer["k"], None)).reshape(t, c.kv_heads, c.head_dim)
        v = f16(oracle.w4a16_linear(n1, *layer["v"], None)).reshape(t, c.kv_heads, c.head_dim)
        q_rot = f16(oracle.rotary_h(q, cos, sin))  # [heads, tokens, d]
        k_rot = f16(oracle.rotary_h(k, cos, sin))
        v_heads = np.ascontiguousarray(v.transpose(1, 0, 2))
        for source, offset in ((k_rot, key_offset), (v_heads, value_offset)):
            oracle.q8_pack(source, slots, pool, _cache_params(c, t, offset))
        repeat = c.q_heads // c.kv_heads
        attention = oracle.attention(q_rot[None], np.repeat(k_rot, repeat, axis=0)[None],
                                     np.repeat(v_heads, repeat, axis=0)[None], causal, 1.0 / math.sqrt(c.head_dim))
        attention = f16(attention[0].transpose(1, 0, 2).reshape(t, -1))  # token-major [tokens, heads * d]
        x_mid = f16(oracle.add(oracle.w4a16_linear(attention, *layer["o"], None), x.astype(np.float32)))
        x = _ffn(c, layer, x_mid)
    final = oracle.rms_norm(x[-1:], weights["final_norm"], c.epsilon)
    logits = oracle.w4a16_linear(final, *weights["lm_head"], None)[0]
    return x, logits, pool


def prefill_first_layer_rows(config, weights, tokens, rows):
    """Rows `rows` of the residual stream after the FIRST layer of a prompt prefill (a one-layer
    chain at lengths where the whole chain is too slow for a CPU check): the keys and values of
    every token are needed, everything else only for the wanted rows."""
    c = config
    t = len(tokens)
    rows = np.asarray(rows)
    layer = weights["layers"][0]
    cos, sin = rope_rows(c, np.arange(t))
    x = weights["embedding"][np.asarray(tokens)]
    n1 = f16(oracle.rms_norm(x, layer["attn_norm"], c.epsilon))
    k = f16(oracle.w4a16_linear(n1, *layer["k"], None)).reshape(t, c.kv_heads, c.head_dim)
    v = f16(oracle.w4a16_linear(n1, *layer["v"], None)).reshape(t, c.kv_heads, c.head_dim)
    k_rot = f16(oracle.rotary_h(k, cos, sin))  # [kv_heads, tokens, d]
    v_heads = np.ascontiguousarray(v.transpose(1, 0, 2))
    q = f16(oracle.w4a16_linear(n1[rows], *layer["q"], None)).reshape(len(rows), c.q_heads, c.head_dim)
    q_rot = f16(oracle.rotary_h(q, cos[rows], sin[rows]))  # [heads, rows, d]
    repeat = c.q_heads // c.kv_heads
    attention = np.empty((len(rows), c.q_heads * c.head_dim), dtype=np.float16)
    for i, row in enumerate(rows):
        visible = np.ones((1, 1, 1, row + 1), dtype=np.float32)
        out = oracle.attention(q_rot[None, :, i:i + 1], np.repeat(k_rot[:, :row + 1], repeat, axis=0)[None],
                               np.repeat(v_heads[:, :row + 1], repeat, axis=0)[None], visible,
                               1.0 / math.sqrt(c.head_dim))
        attention[i] = f16(out[0, :, 0, :].reshape(-1))
    x_mid = f16(oracle.add(oracle.w4a16_linear(attention, *layer["o"], None), x[rows].astype(np.float32)))
    return _ffn(c, layer, x_mid)
