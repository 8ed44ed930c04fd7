"""Llama with the pre-allocated KV cache, attention on the HIP verification kernel.

Module and parameter names match Hugging Face Llama checkpoints (and the reference's
recurrent_drafting/modeling_llama.py), so `from_pretrained` works unchanged.  Projections, MLP and
norms are torch ops (rocBLAS/hipBLASLt GEMMs).  Per forward the bool attention mask is packed to
bits once; per layer the keys and values are appended to the cache in place and
`attention.masked_attention` reads them through strided views -- no repeat_interleave copy, no
additive bias tensor.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
import transformers
from torch import nn
from transformers.activations import ACT2FN
from transformers.modeling_outputs import CausalLMOutput
from transformers.modeling_utils import PreTrainedModel
from transformers.models.llama.configuration_llama import LlamaConfig

from . import _hip, attention, kv_cache
from .packed_rows import PackedRows

KeyValue = Tuple[kv_cache.View, kv_cache.View]


def _fused_weight(owner: nn.Module, name: str, linears) -> torch.Tensor:
    """One (sum of out_features, in_features) weight behind several bias-free Linear layers that
    read the same input.  The layers' own parameters become row slices of it (no second copy,
    checkpoints load and save under the usual names); rebuilt when a parameter was replaced."""
    fused = owner.__dict__.get(name)
    if fused is not None:
        offset, ok = 0, True
        for lin in linears:
            w = lin.weight
            ok = ok and w.dtype == fused.dtype and w.device == fused.device and \
                w.data_ptr() == fused.data_ptr() + offset * fused.element_size()
            offset += w.numel()
        if ok:
            return fused
    assert all(lin.bias is None for lin in linears)
    fused = torch.cat([lin.weight.data for lin in linears], dim=0)
    row = 0
    for lin in linears:
        n = lin.weight.shape[0]
        lin.weight.data = fused[row : row + n]
        row += n
    owner.__dict__[name] = fused
    return fused


def unfuse_weights(model: nn.Module) -> None:
    """Gives every projection its own weight storage again (the state before the first forward).
    After a forward q/k/v_proj and gate/up_proj share one buffer each, which `save_pretrained` with
    safetensors refuses as shared memory; call this before saving.  The next forward fuses again."""
    for module in model.modules():
        for name, group in (("_qkv", ("q_proj", "k_proj", "v_proj")), ("_gate_up", ("gate_proj", "up_proj"))):
            if module.__dict__.pop(name, None) is not None:
                for lin in group:
                    w = getattr(module, lin).weight
                    w.data = w.data.clone()


class LlamaRMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, hidden_states: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        """weight * cast(x * rsqrt(mean(x^2) + eps)), statistics in float32 (modeling_llama.py:27-32).
        With `delta`, hidden_states += delta first, in place, in the same pass (the residual update
        that precedes every norm of a decoder stack)."""
        x = hidden_states
        assert x.stride(-1) == 1 and self.weight.dtype == x.dtype and self.weight.is_contiguous()
        rows = x.numel() // x.shape[-1]
        x2 = x.view(rows, x.shape[-1]) if x.is_contiguous() else x.reshape(rows, x.shape[-1])
        in_place = x2.data_ptr() == x.data_ptr()
        d2 = None
        if delta is not None:
            assert delta.shape == x.shape and delta.dtype == x.dtype and in_place
            d2 = delta.reshape(rows, x.shape[-1])
            assert d2.stride(-1) == 1
        y = torch.empty_like(x2)
        _hip.check(_hip.lib().rd_add_rms_norm(
            _hip.ptr(x2), x2.stride(0), _hip.ptr(d2), 0 if d2 is None else d2.stride(0), _hip.ptr(self.weight),
            _hip.ptr(y), y.stride(0), _hip.ptr(x2) if d2 is not None else None, x2.stride(0),
            _hip.dtype_code(x.dtype), rows, x.shape[-1], float(self.variance_epsilon), _hip.stream()))
        return y.view(x.shape)


class LlamaRotaryEmbedding(nn.Module):
    """cos/sin tables indexed by absolute position; grown on demand (modeling_llama.py:35-72)."""

    def __init__(self, dim: int, max_position_embeddings: int = 2048, base: float = 10000.0,
                 device: Optional[torch.device] = None):
        super().__init__()
        self.dim, self.base = dim, base
        self.register_buffer("inv_freq", self.fresh_inv_freq(device))
        self._build(max_position_embeddings, self.inv_freq.device, torch.get_default_dtype())

    def _build(self, seq_len: int, device, dtype, inv_freq: Optional[torch.Tensor] = None) -> None:
        self.max_seq_len_cached = seq_len
        inv_freq = self.inv_freq if inv_freq is None else inv_freq
        t = torch.arange(seq_len, device=device, dtype=inv_freq.dtype)
        angles = torch.outer(t, inv_freq.to(device))
        table = torch.cat((angles, angles), dim=-1)
        self.cos_cached = table.cos().to(dtype)
        self.sin_cached = table.sin().to(dtype)
        self._cast = {}

    def fresh_inv_freq(self, device=None) -> torch.Tensor:
        return 1.0 / (self.base ** (torch.arange(0, self.dim, 2).float().to(device) / self.dim))

    def forward(self, device: torch.device, dtype: torch.dtype, seq_len: int = 0):
        if self.cos_cached.is_meta:
            # built while transformers constructed the model without memory (from_pretrained of
            # newer releases): the constructor's tables again, from the constructor's float32
            # frequencies (the buffer may have been cast to the checkpoint's dtype since)
            self._build(self.max_seq_len_cached, device, torch.float32, self.fresh_inv_freq(device))
        if seq_len > self.max_seq_len_cached:
            self._build(seq_len, device, dtype)
        key = (device, dtype)
        if key not in self._cast:  # the cast tables are reused by every layer call
            self._cast[key] = (self.cos_cached.to(dtype=dtype).to(device),
                               self.sin_cached.to(dtype=dtype).to(device))
        cos, sin = self._cast[key]
        return cos[:seq_len], sin[:seq_len]


def _rotate_half(x: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids):
    """q, k (B, heads, n, D); cos/sin (positions, D); position_ids (B, n).  NeoX-style rotation."""
    cos = cos[position_ids].unsqueeze(1)
    sin = sin[position_ids].unsqueeze(1)
    return (q * cos) + (_rotate_half(q) * sin), (k * cos) + (_rotate_half(k) * sin)


class LlamaMLP(nn.Module):
    def __init__(self, config: LlamaConfig) -> None:
        super().__init__()
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)
        self.act_fn = ACT2FN[config.hidden_act]
        self._silu = config.hidden_act == "silu"

    def forward(self, x):
        if self._silu:
            # one projection for gate and up, one pass for silu(gate) * up
            weight = _fused_weight(self, "_gate_up", (self.gate_proj, self.up_proj))
            gate_up = nn.functional.linear(x, weight)
            inter = self.gate_proj.out_features
            rows = gate_up.numel() // (2 * inter)
            gu = gate_up.view(rows, 2 * inter)
            act = torch.empty((rows, inter), dtype=x.dtype, device=x.device)
            _hip.check(_hip.lib().rd_silu_mul(
                _hip.ptr(gu), _hip.ptr(gu[:, inter:]), gu.stride(0), _hip.ptr(act), act.stride(0),
                _hip.dtype_code(x.dtype), rows, inter, _hip.stream()))
            return self.down_proj(act.view(*x.shape[:-1], inter))
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


def _rope_theta(config: LlamaConfig) -> float:
    """`rope_theta` of older configs; newer transformers releases keep it in `rope_parameters`."""
    theta = getattr(config, "rope_theta", None)
    if theta is None:
        params = getattr(config, "rope_parameters", None) or {}
        theta = params.get("rope_theta", 10000.0)
    return float(theta)


class LlamaAttention(nn.Module):
    # False: rotation + cache append, then attention (two kernels).  None: one kernel wherever the
    # fused one applies (bf16, head_dim 128, at most 256 new tokens).  Same bits either way.  Measured
    # on the 7B-shaped decode step the fused kernel is 10 us longer than the attention alone and saves
    # the 10-12 us rotation kernel; the step gains between nothing and 2 % from box to box, so the
    # default keeps the two kernels, whose timings can be read one by one.
    fused_rope_attention: Optional[bool] = False

    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = self.hidden_size // self.num_heads
        self.n_kv_heads = config.num_key_value_heads
        self.n_kv_groups = self.num_heads // self.n_kv_heads
        assert self.head_dim * self.num_heads == self.hidden_size
        self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.head_dim, bias=False)
        self.k_proj = nn.Linear(self.hidden_size, self.n_kv_heads * self.head_dim, bias=False)
        self.v_proj = nn.Linear(self.hidden_size, self.n_kv_heads * self.head_dim, bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, self.hidden_size, bias=False)
        self.rotary_emb = LlamaRotaryEmbedding(dim=self.head_dim, base=_rope_theta(config))

    def forward(self, hidden_states: torch.Tensor, position_ids: torch.LongTensor,
                past_key_value: KeyValue, attention_mask: attention.PreparedMask,
                rows: Optional[PackedRows] = None) -> torch.Tensor:
        q_len = position_ids.shape[1]
        # one projection for q, k and v; the three are column slices of its output
        qkv = nn.functional.linear(hidden_states, _fused_weight(self, "_qkv", (self.q_proj, self.k_proj, self.v_proj)))
        nq, nk = self.q_proj.out_features, self.k_proj.out_features
        q, k, v = qkv[..., :nq], qkv[..., nq : nq + nk], qkv[..., nq + nk :]
        cos, sin = self.rotary_emb(v.device, v.dtype, q_len + past_key_value[0].shape[-2])
        # rotation of q and k, append of k and v to the cache, attention (one kernel or two, see
        # fused_rope_attention)
        out = attention.rope_attention(q, k, v, cos, sin, position_ids, past_key_value, attention_mask,
                                       rows=rows, fused=self.fused_rope_attention)  # (B, q_len, hidden)
        return self.o_proj(out)


class LlamaDecoderLayer(nn.Module):
    def __init__(self, config: LlamaConfig) -> None:
        super().__init__()
        self.self_attn = LlamaAttention(config=config)
        self.mlp = LlamaMLP(config)
        self.input_layernorm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)

    def forward(self, hidden_states, position_ids, past_key_value, attention_mask):
        hidden_states, delta = self.forward_deferred(hidden_states, None, position_ids, past_key_value,
                                                     attention_mask)
        hidden_states += delta
        return hidden_states

    def forward_deferred(self, hidden_states, delta, position_ids, past_key_value, attention_mask,
                         rows=None):
        """The layer with its last residual update left to the caller: takes the pending update of
        the layer before (`delta`, or None) and returns (hidden_states, pending update), so that
        every "hidden_states += ..." (modeling_llama.py:196, :198) runs inside the norm that
        follows it."""
        attn = self.self_attn(self.input_layernorm(hidden_states, delta), position_ids, past_key_value,
                              attention_mask, rows)
        return hidden_states, self.mlp(self.post_attention_layernorm(hidden_states, attn))


class LlamaPreTrainedModel(PreTrainedModel):
    config_class = LlamaConfig
    base_model_prefix = "model"

    def _init_weights(self, module: nn.Module) -> None:
        super()._init_weights(module)
        # a checkpoint written by transformers' own Llama has no rotary_emb.inv_freq: what
        # from_pretrained finds missing is what the constructor computes
        if isinstance(module, LlamaRotaryEmbedding) and not module.inv_freq.is_meta:
            with torch.no_grad():
                module.inv_freq.copy_(module.fresh_inv_freq(module.inv_freq.device))


class LlamaModel(LlamaPreTrainedModel):
    def __init__(self, config: LlamaConfig):
        super().__init__(config)
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size, config.pad_token_id)
        self.layers = nn.ModuleList(LlamaDecoderLayer(config) for _ in range(config.num_hidden_layers))
        self.norm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.post_init()

    def get_input_embeddings(self):
        return self.embed_tokens

    def forward(self, input_ids, attention_mask, position_ids, past_key_values,
                rows: Optional[PackedRows] = None) -> torch.Tensor:
        """attention_mask: (B, q, kv) bool, or an attention.PreparedMask built from one.

        With `rows`, only the (B, q) slots that exist pass through the layers and the result is
        (rows.rows, hidden); input_ids, attention_mask and position_ids keep their (B, q) shapes."""
        if not isinstance(attention_mask, attention.PreparedMask):
            attention_mask = attention.prepare(
                attention_mask, fix_empty_rows=False, n_heads=self.config.num_attention_heads,
                kv_shift=_kv_shift(past_key_values))
        if rows is not None:
            input_ids = rows.take_tokens(input_ids)
        hidden_states, delta = self.embed_tokens(input_ids), None
        for layer, key_value in zip(self.layers, past_key_values):
            hidden_states, delta = layer.forward_deferred(hidden_states, delta, position_ids, key_value,
                                                          attention_mask, rows)
        return self.norm(hidden_states, delta)


def _kv_shift(past_key_values) -> Optional[torch.Tensor]:
    """Per-row shift of the cache these views belong to, if its rows are kept in place."""
    owner = past_key_values[0][0]._owner if len(past_key_values) else None
    return owner.shift if owner is not None and owner.rows_in_place else None


class LlamaForCausalLM(LlamaPreTrainedModel):
    # upstream: ["lm_head.weight"] (modeling_llama.py:241); transformers 5 wants the target too
    _tied_weights_keys = (
        {"lm_head.weight": "model.embed_tokens.weight"}
        if int(transformers.__version__.split(".")[0]) >= 5 else ["lm_head.weight"]
    )

    def __init__(self, config):
        super().__init__(config)
        self.model = LlamaModel(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.post_init()

    def get_input_embeddings(self):
        return self.model.embed_tokens

    def get_output_embeddings(self):
        return self.lm_head

    def hidden_states(self, input_ids, attention_mask, position_ids, past_key_values,
                      rows: Optional[PackedRows] = None) -> torch.Tensor:
        """Final-norm hidden states (B, q, hidden), or (rows.rows, hidden) of the slots that
        exist; rows that attend to nothing attend to everything, as the reference arranges on a
        GPU (modeling_llama.py:264-265).  attention_mask: (B, q, kv) bool, or an
        attention.PreparedMask (e.g. from tree_attention.prepare_attention)."""
        prepared = attention_mask if isinstance(attention_mask, attention.PreparedMask) else attention.prepare(
            attention_mask, fix_empty_rows=True, n_heads=self.config.num_attention_heads,
            kv_shift=_kv_shift(past_key_values))
        return self.model(input_ids=input_ids, attention_mask=prepared, position_ids=position_ids,
                          past_key_values=past_key_values, rows=rows)

    def forward(self, input_ids, attention_mask, position_ids, past_key_values) -> CausalLMOutput:
        hidden = self.hidden_states(input_ids, attention_mask, position_ids, past_key_values)
        return CausalLMOutput(logits=self.lm_head(hidden).float(), hidden_states=hidden)
