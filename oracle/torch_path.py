"""Oracle (test infrastructure, never shipped): the whole decode step restated with stock torch ops.

This is the stand-in for "the reference run on this machine": it issues the op sequence of the
reference's files (same dtypes, same temporaries, same rounding points) on whatever device the
tensors live on -- the CPU for the timed CPU baseline, the GPU for parity checks at sizes the CPU
cannot finish.  It owns no weights: it reads them from the model objects it is given (any module
with Hugging Face Llama / ReDrafter parameter names).

  causal_mask, bias            recurrent_drafting/attention.py:12-55, :75-88
  pack, unpack                 recurrent_drafting/tree_attention.py:14-387
  Cache                        recurrent_drafting/kv_cache.py:10-98
  llama_forward                recurrent_drafting/modeling_llama.py:21-276
  beam_search                  recurrent_drafting/modeling_drafter.py:133-232
  greedy_choose, realign       recurrent_drafting/recurrent_drafting.py:114-232, :468-496
  generate_greedy              recurrent_drafting/recurrent_drafting.py:596-705
  sample_choose, residual_distribution, sampling_step, generate_sampling
                               recurrent_drafting/recurrent_drafting.py:75-111, :271-343, :423-430,
                               :499-556 (torch.rand and Categorical.sample supplied by the caller)

Pin status (tests/test_oracle_torch_path.py): pack/unpack/realign/greedy_choose are checked against
tree_oracle / accept_oracle and directly against the reference's literals and vectors; beam_search
against fp_oracle.beam_search_chain; llama_forward, prefill and the loop as a whole are pinned by
the reference's own greedy token streams (tests/golden/reference_vectors.json, "end_to_end": five
tiny float32 models incl. left-padded prompts and pairs whose drafts get accepted), which
generate_greedy reproduces token for token.
The sampling half (tests/test_oracle_sampling_vectors.py) is pinned by vectors the reference
produced with its randomness replaced (torch.rand a recorded tensor / a fixed CPU stream,
Categorical.sample the mode of the probs it is given): sample_choose against
_choose_from_candidates, residual_distribution bit for bit against the probs _prepare_next_input
hands to Categorical, both + realign against _accept_candidate_tokens (whole cache tensors), and
generate_sampling (prefill draw, T != 1, left pads, accepted drafts) against three sampling token
streams of the reference's own loop ("sampling_end_to_end").
Tie rule of the beam search: `tie="stable"` (lowest flat index, the documented rule) or
`tie="topk"` (torch.topk, whatever order it yields; used only when timing the CPU baseline).
"""

from __future__ import annotations

import math
from typing import Generator, Optional, Tuple

import torch
import torch.nn.functional as F

LOG_0 = -50000.0


# ---------------------------------------------------------------------------------------------
# masks
# ---------------------------------------------------------------------------------------------
def causal_mask(padding_mask: torch.Tensor, query_len: int) -> torch.Tensor:
    """Square lower-triangular mask, padded keys cleared, last query_len rows kept."""
    B, kv = padding_mask.shape
    square = torch.ones((kv, kv), dtype=torch.bool, device=padding_mask.device).tril()
    m = square.unsqueeze(0).repeat(B, 1, 1)
    m = m.masked_fill(padding_mask[:, None, :] == 0, False)
    return m[:, kv - query_len :, :]


def rows_without_keys_to_true(mask: torch.Tensor) -> torch.Tensor:
    empty = (mask == 0).sum(dim=-1) == mask.shape[-1]
    return mask.masked_fill(empty[:, :, None], True)


def bias(mask: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    out = torch.zeros(mask.shape, dtype=dtype, device=mask.device)
    return out.masked_fill_(~(mask != 0), torch.finfo(dtype).min)


# ---------------------------------------------------------------------------------------------
# tree packing, tensor formulation
# ---------------------------------------------------------------------------------------------
def pack(beams: torch.Tensor, padding_mask: torch.Tensor):
    """(packed (B,n), unpacker (B,W,L), mask (B,n,prev+n) bool, position_offsets (B,n))."""
    B, W, L = beams.shape
    dev = beams.device
    # owner of every prefix: first beam whose running token equality is still unbroken
    same = (beams[:, :, None, :] == beams[:, None, :, :]).long()
    unbroken = same.cumsum(dim=3) == torch.arange(1, L + 1, device=dev)
    owner = unbroken.long().argmax(dim=2)  # (B,W,L)
    own = owner == torch.arange(W, device=dev)[None, :, None]
    # unpacker: start of the owner's segment plus position inside it
    n_own = own.sum(dim=-1)
    start = n_own.cumsum(dim=-1) - n_own
    seg = start.gather(1, owner.view(B, -1)).view(B, W, L)
    earlier = torch.arange(L, device=dev)[:, None] > torch.arange(L, device=dev)[None, :]
    unpacker = seg + ((seg[:, :, :, None] == seg[:, :, None, :]) & earlier).sum(dim=-1)
    # pack: one vector over the batch, per-row windows clamped to its end
    where = own.view(B, -1).nonzero()
    chosen = beams.reshape(B, -1)[where[:, 0], where[:, 1]]
    n_sel = own.view(B, -1).sum(dim=1)
    n = int(n_sel.max())
    first = n_sel.cumsum(0) - n_sel
    window = (first[:, None] + torch.arange(n, device=dev)).clamp(max=chosen.numel() - 1)
    packed = chosen[window]
    flat_index = where[:, 1][window]  # beam*L + position of every packed slot
    # mask: prefix part from the padding mask, tree part scattered per packed slot
    prev = padding_mask.shape[1]
    ext = torch.cat([padding_mask != 0, torch.ones((B, n), dtype=torch.bool, device=dev)], dim=1)
    full = causal_mask(ext, prev + n).clone()
    beam_of = flat_index // L
    pos_of = flat_index % L
    targets = unpacker.gather(1, beam_of[:, :, None].expand(B, n, L))  # (B,n,L)
    allowed = torch.arange(L, device=dev)[None, None, :] <= pos_of[:, :, None]
    tree = torch.zeros((B, n, n), dtype=torch.bool, device=dev).scatter_(2, targets, allowed)
    full[:, prev:, prev:] = tree
    return packed, unpacker, full[:, -n:, :], pos_of


def unpack(packed: torch.Tensor, unpacker: torch.Tensor) -> torch.Tensor:
    B, W, L = unpacker.shape
    idx = unpacker.view(B, W * L, 1).expand(-1, -1, packed.shape[2])
    return packed.gather(1, idx).reshape(B, W, L, -1)


# ---------------------------------------------------------------------------------------------
# KV cache
# ---------------------------------------------------------------------------------------------
class Cache:
    def __init__(self, batch, max_length, n_layers, n_heads, head_dim, dtype, device):
        self.data = torch.zeros((n_layers, 2, batch, n_heads, max_length, head_dim), dtype=dtype, device=device)
        self.length = [[0, 0] for _ in range(n_layers)]

    def append(self, layer: int, kv: int, new: torch.Tensor) -> torch.Tensor:
        at = self.length[layer][kv]
        n = new.shape[2]
        assert at + n <= self.data.shape[4]
        self.data[layer, kv, :, :, at : at + n, :] = new
        self.length[layer][kv] = at + n
        return self.data[layer, kv, :, :, : at + n, :]

    def set_length(self, n: int) -> None:
        for pair in self.length:
            pair[0] = pair[1] = n

    def unpack(self, prev: int, unpacker: torch.Tensor) -> None:
        """Gather with a fully expanded index, clone, write back (the reference's traffic)."""
        B, W, L = unpacker.shape
        n_layers, _, _, H, _, D = self.data.shape
        idx = (prev + unpacker.view(1, 1, B, 1, W * L, 1)).expand(n_layers, 2, -1, H, -1, D)
        self.data[:, :, :, :, prev : prev + W * L, :] = torch.gather(self.data, 4, idx).clone()
        self.set_length(prev + W * L)


# ---------------------------------------------------------------------------------------------
# Llama forward with an additive bias and stock SDPA
# ---------------------------------------------------------------------------------------------
def _rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    y = x.to(torch.float32)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    return weight * y.to(x.dtype)


def _rope_tables(head_dim: int, base: float, n_pos: int, device, dtype):
    inv = 1.0 / (base ** (torch.arange(0, head_dim, 2, device=device).float() / head_dim))
    ang = torch.outer(torch.arange(n_pos, device=device, dtype=inv.dtype), inv)
    emb = torch.cat((ang, ang), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def _rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return (x * cos) + (rot * sin)


def _theta(cfg) -> float:
    t = getattr(cfg, "rope_theta", None)
    if t is None:
        t = (getattr(cfg, "rope_parameters", None) or {}).get("rope_theta", 10000.0)
    return float(t)


def llama_forward(llm, input_ids, mask, position_ids, cache: Cache, on_gpu_semantics: bool = True):
    """Returns (logits float32 (B,q,V), hidden (B,q,hid)).  mask: (B,q,kv) bool."""
    cfg = llm.config
    H, Hkv = cfg.num_attention_heads, cfg.num_key_value_heads
    D = cfg.hidden_size // H
    if on_gpu_semantics:
        mask = rows_without_keys_to_true(mask)
    x = llm.model.embed_tokens(input_ids)
    attn_bias = bias(mask.unsqueeze(1), x.dtype)
    B, q_len = input_ids.shape
    kv_len = mask.shape[-1]
    cos_t, sin_t = _rope_tables(D, _theta(cfg), max(kv_len, 2048), x.device, x.dtype)
    cos = cos_t[position_ids].unsqueeze(1)
    sin = sin_t[position_ids].unsqueeze(1)
    for li, layer in enumerate(llm.model.layers):
        att = layer.self_attn
        h = _rms_norm(x, layer.input_layernorm.weight, cfg.rms_norm_eps)
        q = F.linear(h, att.q_proj.weight).view(B, q_len, H, D).transpose(1, 2)
        k = F.linear(h, att.k_proj.weight).view(B, q_len, Hkv, D).transpose(1, 2)
        v = F.linear(h, att.v_proj.weight).view(B, q_len, Hkv, D).transpose(1, 2)
        q, k = _rope(q, cos, sin), _rope(k, cos, sin)
        keys = cache.append(li, 0, k)
        values = cache.append(li, 1, v)
        keys = keys.repeat_interleave(H // Hkv, dim=1)
        values = values.repeat_interleave(H // Hkv, dim=1)
        o = F.scaled_dot_product_attention(q, keys, values, attn_mask=attn_bias)
        o = o.transpose(1, 2).contiguous().reshape(B, q_len, H * D)
        x = x + F.linear(o, att.o_proj.weight)
        h = _rms_norm(x, layer.post_attention_layernorm.weight, cfg.rms_norm_eps)
        mlp = layer.mlp
        x = x + F.linear(F.silu(F.linear(h, mlp.gate_proj.weight)) * F.linear(h, mlp.up_proj.weight),
                         mlp.down_proj.weight)
    x = _rms_norm(x, llm.model.norm.weight, cfg.rms_norm_eps)
    return F.linear(x, llm.lm_head.weight).float(), x


# ---------------------------------------------------------------------------------------------
# drafter beam search
# ---------------------------------------------------------------------------------------------
def top_k_filter(x: torch.Tensor, k: int = 50, fill: float = LOG_0) -> torch.Tensor:
    k = min(k, x.shape[-1])
    kth = torch.topk(x, k).values[..., -1:]
    return x.masked_fill(x < kth, fill)


def drafter_logits(drafter, x: torch.Tensor) -> torch.Tensor:
    if hasattr(drafter, "input_proj"):
        x = drafter.input_proj(x)
    y = drafter.lm_head(x)
    y = y - y.max(dim=-1, keepdim=True).values
    return top_k_filter(y)


def beam_search(drafter, embeddings, prompt_state, init_token, width: int, length: int,
                tie: str = "stable", want_log_probs: bool = True):
    B, hid = prompt_state.shape
    dev = prompt_state.device
    V = embeddings.num_embeddings
    score = torch.tensor([0.0] + [LOG_0] * (width - 1), device=dev).repeat(B, 1)
    context = prompt_state[:, None, :].repeat(1, width, 1)
    beams = init_token[:, None, None].repeat(1, width, 1)
    state = torch.zeros((B, width, hid), device=dev, dtype=prompt_state.dtype)
    hist = torch.zeros((B, width, 0, V), device=dev)
    rows = torch.arange(B, device=dev)[:, None]
    for _ in range(length - 1):
        last = embeddings(beams[..., -1])
        state = F.silu(drafter.rnn_w(last) + drafter.rnn_u(state)) if drafter.config.rnn else last + state
        logp = drafter_logits(drafter, torch.cat([context, state], dim=-1)).log_softmax(dim=-1)
        joint = (logp + score[:, :, None]).reshape(B, width * V)
        if tie == "stable":
            order = torch.sort(joint, dim=-1, descending=True, stable=True)
            score, flat = order.values[:, :width], order.indices[:, :width]
        else:
            score, flat = torch.topk(joint, k=width, dim=-1)
        tok, parent = flat % V, flat // V
        beams = torch.cat([beams[rows, parent], tok[:, :, None]], dim=-1)
        state = state[rows, parent]
        if want_log_probs:
            hist = torch.cat([hist[rows, parent], logp[rows, parent][:, :, None]], dim=2)
    return beams, (hist if want_log_probs else None)


# ---------------------------------------------------------------------------------------------
# acceptance and re-alignment
# ---------------------------------------------------------------------------------------------
def count_left_pads(ids: torch.Tensor, pad: int) -> torch.Tensor:
    return (ids == pad).long().cumprod(dim=-1).sum(dim=-1)


def greedy_choose(beams: torch.Tensor, llm_tokens: torch.Tensor):
    agree = (beams[:, :, 1:] == llm_tokens[:, :, :-1]).long()
    n = agree.cumprod(dim=-1).sum(dim=-1)
    best = n.max(dim=-1)
    return best.values, best.indices


def realign(input_ids, n_tokens, seq_in_beam, beams, cache: Cache, pad: int) -> torch.Tensor:
    """Cache must be unpacked.  Beam rows copied behind the prefix, whole live cache cloned, every
    row copied to its right-aligned place; ids rebuilt the same way."""
    B, W, L = beams.shape
    prev = input_ids.shape[1]
    pads = count_left_pads(input_ids, pad)
    n_new = n_tokens + 1
    seq_len = prev - pads + n_new
    M = int(seq_len.max())
    new_pads = M - seq_len
    n_layers, _, _, H, _, D = cache.data.shape
    rows = torch.arange(B, device=input_ids.device)
    cache.set_length(prev)
    region = cache.data[:, :, :, :, prev : prev + W * L, :]
    for li in range(n_layers):
        for kv in range(2):
            cand = region[li, kv].reshape(B * H, W, L, D)
            pick = cand[torch.arange(B * H, device=cand.device), seq_in_beam[:, None].expand(B, H).reshape(-1)]
            cache.append(li, kv, pick.reshape(B, H, L, D))
    # the reference slices dimension 3 (heads) with the sequence length here, which keeps every
    # head: the whole allocation is cloned, not just the live prefix (recurrent_drafting.py:201)
    snapshot = cache.data[:, :, :, : prev + L, :].clone()
    for b in range(B):
        lo, hi = int(pads[b]), prev + int(n_new[b])
        cache.data[:, :, b, :, int(new_pads[b]) : M, :] = snapshot[:, :, b, :, lo:hi, :]
    chosen = beams[rows, seq_in_beam]
    ids = torch.full((B, M), pad, dtype=input_ids.dtype, device=input_ids.device)
    for b in range(B):
        a = int(new_pads[b])
        e = a + prev - int(pads[b])
        ids[b, a:e] = input_ids[b, int(pads[b]) :]
        ids[b, e : e + int(n_new[b])] = chosen[b, : int(n_new[b])]
    cache.set_length(M)
    return ids


# ---------------------------------------------------------------------------------------------
# decode loop
# ---------------------------------------------------------------------------------------------
def prefill(llm, input_ids, cache: Cache, pad: int):
    S = input_ids.shape[1]
    mask = causal_mask(input_ids != pad, S)
    pos = torch.arange(S, device=input_ids.device).expand(input_ids.shape) - count_left_pads(input_ids, pad)[:, None]
    logits, hidden = llama_forward(llm, input_ids, mask, pos, cache)
    return hidden[:, -1, :], top_k_filter(logits[:, -1, :]).argmax(dim=-1)


def greedy_step(llm, drafter, input_ids, context, init_tokens, cache: Cache, width, length, pad,
                tie: str = "stable"):
    """One draft / verify / accept step.  Returns (context, input_ids, next_tokens, n_tokens, beams)."""
    beams, _ = beam_search(drafter, llm.model.embed_tokens, context, init_tokens, width, length,
                           tie=tie, want_log_probs=False)
    packed, unpacker, mask, offsets = pack(beams, (input_ids != pad).to(input_ids.dtype))
    prev = input_ids.shape[1]
    pos = (prev - count_left_pads(input_ids, pad))[:, None] + offsets
    logits, hidden = llama_forward(llm, packed, mask, pos, cache)
    logits = top_k_filter(logits)
    hidden = unpack(hidden, unpacker)
    logits = unpack(logits, unpacker)
    cache.unpack(prev, unpacker)
    llm_tokens = logits.argmax(dim=-1)
    n_tokens, seq_in_beam = greedy_choose(beams, llm_tokens)
    input_ids = realign(input_ids, n_tokens, seq_in_beam, beams, cache, pad)
    rows = torch.arange(beams.shape[0], device=beams.device)
    next_tokens = llm_tokens[rows, seq_in_beam, n_tokens]
    context = hidden[rows, seq_in_beam, n_tokens]
    return context, input_ids, next_tokens, n_tokens, beams


def sample_choose(beams, log_p_llm, log_q_drafter, uniforms):
    """recurrent_drafting.py:532-556 with the uniforms supplied by the caller."""
    tok = beams[..., 1:, None]
    q = log_q_drafter.gather(-1, tok).squeeze(-1)
    p = log_p_llm[:, :, :-1, :].gather(-1, tok).squeeze(-1)
    ok = uniforms < torch.exp(p - q)
    run = (ok.long().cumsum(-1) == torch.arange(1, ok.shape[-1] + 1, device=ok.device)).sum(-1)
    best = run.max(dim=-1)
    return best.values, best.indices


def residual_distribution(log_q_drafter, log_p_llm, seq_in_beam, n_tokens):
    """Unnormalised next-token distribution (recurrent_drafting.py:304-339)."""
    B, W, Lm1, V = log_q_drafter.shape
    rows = torch.arange(B, device=log_q_drafter.device)
    q_sel, p_sel = log_q_drafter[rows, seq_in_beam], log_p_llm[rows, seq_in_beam]
    whole = (n_tokens == Lm1)[:, None]
    idx = n_tokens - (n_tokens == Lm1).long()
    resid = torch.relu(torch.exp(p_sel[rows, idx]) - torch.exp(q_sel[rows, idx]))
    return torch.where(whole, torch.exp(p_sel[:, -1]), resid)


def sampling_step(llm, drafter, input_ids, context, init_tokens, cache: Cache, width, length, pad,
                  temperature, draw_uniforms, draw_token, tie: str = "stable"):
    """One speculative-sampling step (recurrent_drafting.py:75-111, :437-465).  draw_uniforms(shape)
    and draw_token(probs) stand in for torch.rand and Categorical(probs).sample()."""
    beams, log_q = beam_search(drafter, llm.model.embed_tokens, context, init_tokens, width, length, tie=tie)
    packed, unpacker, mask, offsets = pack(beams, (input_ids != pad).to(input_ids.dtype))
    prev = input_ids.shape[1]
    pos = (prev - count_left_pads(input_ids, pad))[:, None] + offsets
    logits, hidden = llama_forward(llm, packed, mask, pos, cache)
    logits = unpack(top_k_filter(logits), unpacker)
    hidden = unpack(hidden, unpacker)
    cache.unpack(prev, unpacker)
    log_p = (logits / temperature).log_softmax(dim=-1)
    n_tokens, seq_in_beam = sample_choose(beams, log_p, log_q, draw_uniforms(log_q.shape[:3]))
    input_ids = realign(input_ids, n_tokens, seq_in_beam, beams, cache, pad)
    next_tokens = draw_token(residual_distribution(log_q, log_p, seq_in_beam, n_tokens))
    rows = torch.arange(beams.shape[0], device=beams.device)
    context = hidden[rows, seq_in_beam, n_tokens]
    return context, input_ids, next_tokens, n_tokens, beams


def generate_greedy(llm, drafter, input_ids, max_length: int, width: int, length: int, pad: int = 0,
                    eos: Optional[int] = 1, tie: str = "stable") -> Generator[Tuple[torch.Tensor, torch.Tensor], None, None]:
    """Yields (output tokens (B, <=max_length), n_tokens_in_seq (B,)) after every step."""
    with torch.inference_mode():
        B, S = input_ids.shape
        cfg = llm.config
        cache = Cache(B, max_length + width * length, cfg.num_hidden_layers, cfg.num_key_value_heads,
                      cfg.hidden_size // cfg.num_attention_heads, llm.lm_head.weight.dtype, input_ids.device)
        context, tokens = prefill(llm, input_ids, cache, pad)
        seq_len = S
        while seq_len < max_length:
            context, input_ids, tokens, n_tokens, _ = greedy_step(
                llm, drafter, input_ids, context, tokens, cache, width, length, pad, tie)
            out = torch.cat((input_ids, tokens[:, None]), dim=-1)
            seq_len = out.shape[1]
            yield out[:, :max_length], n_tokens
            if eos is not None and bool(((out[:, S:] == eos).sum(dim=-1) > 0).all()):
                break


def generate_sampling(llm, drafter, input_ids, max_length: int, width: int, length: int, temperature: float,
                      draw_uniforms, draw_token, pad: int = 0, eos: Optional[int] = 1, tie: str = "stable"):
    """Speculative-sampling decode loop; yields (output tokens, n_tokens_in_seq) per step."""
    with torch.inference_mode():
        B, S = input_ids.shape
        cfg = llm.config
        cache = Cache(B, max_length + width * length, cfg.num_hidden_layers, cfg.num_key_value_heads,
                      cfg.hidden_size // cfg.num_attention_heads, llm.lm_head.weight.dtype, input_ids.device)
        mask = causal_mask(input_ids != pad, S)
        pos = torch.arange(S, device=input_ids.device).expand(input_ids.shape) - count_left_pads(input_ids, pad)[:, None]
        logits, hidden = llama_forward(llm, input_ids, mask, pos, cache)
        context = hidden[:, -1, :]
        tokens = draw_token(torch.softmax(top_k_filter(logits[:, -1, :]) / temperature, dim=-1))
        seq_len = S
        while seq_len < max_length:
            context, input_ids, tokens, n_tokens, _ = sampling_step(
                llm, drafter, input_ids, context, tokens, cache, width, length, pad, temperature,
                draw_uniforms, draw_token, tie)
            out = torch.cat((input_ids, tokens[:, None]), dim=-1)
            seq_len = out.shape[1]
            yield out[:, :max_length], n_tokens
            if eos is not None and bool(((out[:, S:] == eos).sum(dim=-1) > 0).all()):
                break
