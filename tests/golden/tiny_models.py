"""Deterministic tiny Llama + drafter weights shared by the fixture generator and the tests.

Configuration 1 of the benchmark plan: Llama with 2 layers, hidden 128, 4 heads x 32, FFN 344,
vocabulary 1000, float32; drafter with one residual block, hidden 128, exit_dim 256, recurrent
state on.  Weights are N(0, 0.02) drawn on the CPU with torch.manual_seed(seed) in sorted-name
order (norm gains are 1, biases drawn like weights), so every machine with the same torch builds
the same tensors.
"""

from __future__ import annotations

from typing import Dict, Tuple

import torch

LLAMA = dict(vocab_size=1000, hidden_size=128, intermediate_size=344, num_hidden_layers=2,
             num_attention_heads=4, num_key_value_heads=4, rms_norm_eps=1e-6, hidden_act="silu",
             pad_token_id=0, max_position_embeddings=2048)
DRAFTER = dict(vocab_size=1000, hidden_size=128, exit_dim=256, num_draft_layers=1, rnn=True)


def llama_shapes(c=LLAMA) -> Dict[str, Tuple[int, ...]]:
    h, f, v = c["hidden_size"], c["intermediate_size"], c["vocab_size"]
    hk = c["num_key_value_heads"] * (h // c["num_attention_heads"])
    shapes = {"model.embed_tokens.weight": (v, h), "model.norm.weight": (h,), "lm_head.weight": (v, h)}
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes.update({
            p + "self_attn.q_proj.weight": (h, h), p + "self_attn.k_proj.weight": (hk, h),
            p + "self_attn.v_proj.weight": (hk, h), p + "self_attn.o_proj.weight": (h, h),
            p + "mlp.gate_proj.weight": (f, h), p + "mlp.up_proj.weight": (f, h),
            p + "mlp.down_proj.weight": (h, f),
            p + "input_layernorm.weight": (h,), p + "post_attention_layernorm.weight": (h,),
        })
    return shapes


def drafter_shapes(c=DRAFTER) -> Dict[str, Tuple[int, ...]]:
    h, e, v = c["hidden_size"], c["exit_dim"], c["vocab_size"]
    shapes = {}
    for i in range(c["num_draft_layers"]):
        shapes[f"lm_head.{i}.linear.weight"] = (e, e)
        shapes[f"lm_head.{i}.linear.bias"] = (e,)
    shapes[f"lm_head.{c['num_draft_layers']}.weight"] = (v, e)
    if 2 * h != e:
        shapes["input_proj.weight"] = (e, 2 * h)
        shapes["input_proj.bias"] = (e,)
    if c["rnn"]:
        shapes.update({"rnn_u.weight": (h, h), "rnn_u.bias": (h,), "rnn_w.weight": (h, h)})
    return shapes


def draw(shapes: Dict[str, Tuple[int, ...]], seed: int, std: float = 0.02) -> Dict[str, torch.Tensor]:
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = {}
    for name in sorted(shapes):
        if name.endswith("layernorm.weight") or name == "model.norm.weight":
            out[name] = torch.ones(shapes[name])
        else:
            out[name] = torch.randn(shapes[name], generator=gen) * std
    return out


def prompt(batch: int, length: int, vocab: int, seed: int, left_pads=()) -> torch.Tensor:
    """Token ids uniform over [1, vocab) (never the pad id 0), optional left padding per row."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    ids = torch.randint(1, vocab, (batch, length), generator=gen)
    for b, n in enumerate(left_pads):
        ids[b, :n] = 0
    return ids


def markov(seed: int, gain: float = 40.0, llama_cfg=LLAMA, drafter_cfg=DRAFTER, mix: float = 0.0):
    """(llama_state, drafter_state) of a toy pair in which the drafter usually agrees with the LLM,
    so that decoding accepts drafted tokens: embeddings are non-negative, the drafter decodes
    silu(gain * embedding) with the LLM's own lm_head, and the attention and MLP outputs of the LLM
    are scaled by `mix`.  mix = 0 (the default): the residual stream is the token embedding, the
    next token depends on the last token only and the drafter is nearly always right; with a small
    mix the context moves the LLM's choice now and then, so accepted lengths become ragged and
    the attention output matters for the tokens."""
    llama = draw(llama_shapes(llama_cfg), seed)
    llama["model.embed_tokens.weight"] = llama["model.embed_tokens.weight"].abs()
    for name in llama:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            llama[name] = llama[name] * mix
    drafter = draw(drafter_shapes(drafter_cfg), seed + 1000)
    h = drafter_cfg["hidden_size"]
    drafter["rnn_w.weight"] = torch.eye(h) * gain
    drafter["rnn_u.weight"] = torch.zeros(h, h)
    drafter["rnn_u.bias"] = torch.zeros(h)
    drafter["lm_head.0.linear.weight"] = torch.zeros_like(drafter["lm_head.0.linear.weight"])
    drafter["lm_head.0.linear.bias"] = torch.full_like(drafter["lm_head.0.linear.bias"], -30.0)
    drafter["lm_head.1.weight"] = torch.cat(
        [torch.zeros(drafter_cfg["vocab_size"], h), llama["lm_head.weight"] * 8.0], dim=1)
    return llama, drafter
