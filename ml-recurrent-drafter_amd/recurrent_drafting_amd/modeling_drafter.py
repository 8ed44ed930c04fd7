"""Recurrent drafter head and its beam search.

Module and parameter names follow the reference's recurrent_drafting/modeling_drafter.py, so its
checkpoints load.  The dense layers stay on torch (rocBLAS/hipBLASLt GEMMs); everything after the
vocabulary GEMM of one beam-search iteration -- max subtraction, top-50 filter, log-softmax, beam
score, top-W over width*vocab, parent/token split, beam gather -- is one call of rd_beam_topk.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import transformers

from . import _hip, configuration_drafter, tree_attention

LOG_0 = -50000.0
LOG_1 = 0.0
TOP_K = 50


@dataclass
class BeamShape:
    width: int
    length: int


def register_auto_models() -> None:
    cfg = configuration_drafter.DrafterConfig
    transformers.AutoConfig.register(model_type=cfg.model_type, config=cfg)
    transformers.AutoModel.register(config_class=cfg, model_class=Drafter)


class ResBlock(torch.nn.Module):
    def __init__(self, cfg: configuration_drafter.DrafterConfig):
        super().__init__()
        self.linear = torch.nn.Linear(cfg.exit_dim, cfg.exit_dim, bias=True)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return x + torch.nn.functional.silu(self.linear(x))


def silu_add(x: torch.Tensor, z: torch.Tensor, mode: int, also: Optional[torch.Tensor] = None) -> torch.Tensor:
    """mode 0: x + silu(z); mode 1: silu(x + z).  x and z (..., cols) of one dtype with contiguous
    columns and a common row layout; `also`, a (..., cols) view of the same leading shape whose
    rows may be strided, receives a second copy of the result."""
    cols = x.shape[-1]
    assert x.shape == z.shape and x.dtype == z.dtype
    x2, z2 = x.reshape(-1, cols), z.reshape(-1, cols)
    assert x2.stride(1) == 1 and z2.stride(1) == 1
    out = torch.empty((x2.shape[0], cols), dtype=x.dtype, device=x.device)
    y2 = None
    if also is not None:
        assert also.shape == x.shape and also.dtype == x.dtype and also.stride(-1) == 1
        y2 = also.view(-1, cols)  # (a view: the rows of `also` must be evenly strided)
    _hip.check(_hip.lib().rd_silu_add(
        _hip.ptr(x2), x2.stride(0), _hip.ptr(z2), z2.stride(0), _hip.ptr(out), out.stride(0),
        _hip.ptr(y2), 0 if y2 is None else y2.stride(0), mode, _hip.dtype_code(x.dtype),
        x2.shape[0], cols, _hip.stream()))
    return out.view(x.shape)


def _gather_beams(x: torch.Tensor, selected_beams: torch.Tensor) -> torch.Tensor:
    """x (B, W, ...) re-ordered along dim 1 by selected_beams (B, W) (modeling_drafter.py:42-53)."""
    B, W = x.shape[0], x.shape[1]
    out = tree_attention.gather_rows(x.reshape(B, W, -1), selected_beams.to(torch.long))
    return out.view(x.shape)


def _add_decoding_dim(x: torch.Tensor, beam_width: int) -> torch.Tensor:
    """(B, ...) -> (B, beam_width, ...) by repetition (modeling_drafter.py:56-60)."""
    return x.unsqueeze(1).repeat_interleave(beam_width, dim=1)


def maintain_logits(logits: torch.Tensor) -> torch.Tensor:
    """Row maximum subtracted (modeling_drafter.py:63-77).  The beam search fuses this step."""
    return logits - logits.amax(dim=-1, keepdim=True)


def warp_logits(logits: torch.Tensor, top_k: int = TOP_K, mask_value: float = LOG_0) -> torch.Tensor:
    """Everything below the row's top_k-th largest value becomes mask_value
    (modeling_drafter.py:80-99).  The beam search and the greedy decode loop never materialise
    this tensor; the function is kept for callers that want it."""
    top_k = min(top_k, logits.size(-1))
    kth = torch.topk(logits, top_k).values[..., -1:]
    return logits.masked_fill(logits < kth, mask_value)


def beam_topk_step(
    logits: torch.Tensor,
    log_p_beam: torch.Tensor,
    beams: torch.Tensor,
    want_log_probs: bool,
    force_fallback: bool = False,
):
    """One fused post-GEMM iteration.  logits (B, W, V); log_p_beam (B, W) f32; beams (B, W, t).

    Returns (new_log_p_beam, tokens, parents, new_beams (B, W, t+1), log_p_new_token or None)."""
    B, W, V = logits.shape
    assert log_p_beam.dtype == torch.float32 and log_p_beam.shape == (B, W)
    assert beams.dtype == torch.long and beams.shape[:2] == (B, W)
    if logits.stride(1) == 0 and logits.stride(2) == 1 and logits.stride(0) >= V \
            and (logits.stride(0) * logits.element_size()) % 16 == 0 and logits.data_ptr() % 16 == 0:
        # one row per batch row shown W times (the first iteration): the kernel reads it in place
        x, row_stride, batch_stride = logits, 0, logits.stride(0)
    else:
        x = logits.reshape(B * W, V)
        if x.stride(0) < V:  # rows shown several times some other way: the kernel wants real rows
            x = x.contiguous()
        x = _hip.aligned_rows(x)
        row_stride, batch_stride = x.stride(0), 0
    beams = beams.contiguous()
    log_p_beam = log_p_beam.contiguous()
    t = beams.shape[2]
    dev = logits.device
    lib = _hip.lib()
    new_lpb = torch.empty((B, W), dtype=torch.float32, device=dev)
    tok_par = torch.empty((2, B, W), dtype=torch.long, device=dev)
    new_beams = torch.empty((B, W, t + 1), dtype=torch.long, device=dev)
    logp = torch.empty((B, W, V), dtype=torch.float32, device=dev) if want_log_probs else None
    ws_bytes = lib.rd_beam_topk_workspace_bytes(B, W)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    _hip.check(
        lib.rd_beam_topk(
            _hip.ptr(x), _hip.dtype_code(x.dtype), row_stride, batch_stride, B, W, V, _hip.ptr(log_p_beam),
            TOP_K, LOG_0, _hip.ptr(beams), t, _hip.ptr(new_lpb), _hip.ptr(tok_par[0]),
            _hip.ptr(tok_par[1]), _hip.ptr(new_beams), _hip.ptr(logp), V, _hip.ptr(ws), ws.numel(),
            int(force_fallback), _hip.stream(),
        )
    )
    return new_lpb, tok_par[0], tok_par[1], new_beams, logp


def beam_init(prompt_state: torch.Tensor, init_token: torch.Tensor, width: int, state_rows: int):
    """The state the beam search starts from (modeling_drafter.py:170-189): log_p_beam (B, W) float32
    with only beam 0 alive, beams (B, W, 1) holding the init token, the (B, W, 2*hidden) input of the
    head with its context half filled in, and the zero state of the first `state_rows` beams."""
    B, hidden = prompt_state.shape
    dev, dt = prompt_state.device, prompt_state.dtype
    if prompt_state.stride(1) != 1:
        prompt_state = prompt_state.contiguous()
    init_token = init_token.contiguous()
    log_p_beam = torch.empty((B, width), dtype=torch.float32, device=dev)
    beams = torch.empty((B, width, 1), dtype=torch.long, device=dev)
    head_in = torch.empty((B, width, 2 * hidden), dtype=dt, device=dev)
    state = torch.empty((B, state_rows, hidden), dtype=dt, device=dev)
    esize = prompt_state.element_size()
    _hip.check(
        _hip.lib().rd_beam_init(
            _hip.ptr(prompt_state), prompt_state.stride(0) * esize, _hip.ptr(init_token), B, width, hidden * esize,
            LOG_0, _hip.ptr(log_p_beam), _hip.ptr(beams), _hip.ptr(head_in), 2 * hidden * esize, _hip.ptr(state),
            state_rows, _hip.stream(),
        )
    )
    return log_p_beam, beams, head_in, state


class Drafter(transformers.PreTrainedModel):
    config_class = configuration_drafter.DrafterConfig
    # False computes the first beam-search iteration for all W (identical) beams, as upstream does
    first_iteration_once = True

    def __init__(self, cfg: configuration_drafter.DrafterConfig):
        super().__init__(cfg)
        self.config = cfg
        if 2 * cfg.hidden_size != cfg.exit_dim:  # optional projection of [context, state]
            self.input_proj = torch.nn.Linear(2 * cfg.hidden_size, cfg.exit_dim, bias=True)
        blocks = [ResBlock(cfg) for _ in range(cfg.num_draft_layers)]
        self.lm_head = torch.nn.Sequential(
            *blocks, torch.nn.Linear(cfg.exit_dim, cfg.vocab_size, bias=False)
        )
        if cfg.rnn:
            self.rnn_u = torch.nn.Linear(cfg.hidden_size, cfg.hidden_size, bias=True)
            self.rnn_w = torch.nn.Linear(cfg.hidden_size, cfg.hidden_size, bias=False)
        # transformers' bookkeeping for save_pretrained / from_pretrained (newer releases refuse to
        # load a model whose constructor skipped it); the layers keep torch's own initialisation,
        # as upstream's do (modeling_drafter.py:104-125 never runs transformers' initialiser)
        self.post_init()

    def _init_weights(self, module: torch.nn.Module) -> None:
        return

    def raw_logits(self, x: torch.Tensor) -> torch.Tensor:
        """Vocabulary logits of [context, state] before any normalisation: `self.lm_head`, with
        the sum and the activation of every ResBlock (modeling_drafter.py:38-39) in one kernel."""
        x = self.input_proj(x) if hasattr(self, "input_proj") else x
        *blocks, head = self.lm_head
        for block in blocks:
            x = silu_add(x, block.linear(x), mode=0)
        return head(x)

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        """Logits with the row maximum at zero and everything below the top 50 at LOG_0
        (modeling_drafter.py:127-131)."""
        return warp_logits(maintain_logits(self.raw_logits(x)))

    def beam_search_candidates(
        self,
        prompt_state: torch.Tensor,
        init_token: torch.Tensor,
        embeddings: torch.nn.Embedding,
        beam_shape: BeamShape = BeamShape(10, 4),
        return_log_probs: bool = True,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """beams (B, W, L) int64 and, unless return_log_probs is False, the drafter's
        log-probabilities (B, W, L-1, V) float32 of every drafted position
        (modeling_drafter.py:133-232).  Greedy decoding never reads the log-probabilities."""
        assert init_token.dtype == torch.long
        assert prompt_state.ndim == 2
        assert init_token.ndim == 1
        assert beam_shape.length > 1
        B, hidden = prompt_state.shape
        W, L = beam_shape.width, beam_shape.length
        V = embeddings.num_embeddings
        dev = prompt_state.device

        # only beam 0 is alive at the start, so the first iteration fans out from it alone.
        # [context, state] is the input of the head (modeling_drafter.py:199): the context half is
        # written once, here, the state half by the kernel that forms the state.  Scores, first
        # tokens, context halves and the zero state come from one launch.
        first_rows = 1 if self.first_iteration_once else W  # beams whose state the first iteration reads
        log_p_beam, beams, head_in, state = beam_init(prompt_state, init_token, W, first_rows)
        newest = init_token.view(B, 1) if first_rows == 1 else beams[:, :, 0]  # (B, rows of the first iteration)
        step_log_probs: List[torch.Tensor] = []
        step_parents: List[torch.Tensor] = []

        for it in range(L - 1):
            # In the first iteration every beam of a row holds the same token, state and context
            # (modeling_drafter.py:170-189), so the W rows of logits are W copies of one row:
            # that row is computed once per batch row and shown W times.
            rows = 1 if it == 0 and self.first_iteration_once else W
            # (the newest token of every beam, from a contiguous tensor: beams[:, :rows, -1] is a
            # strided view, which the lookup would copy first)
            last = embeddings(newest[:, :rows])
            if self.config.rnn:
                state = silu_add(self.rnn_w(last), self.rnn_u(state[:, :rows]), mode=1,
                                 also=head_in[:, :rows, hidden:])
            else:
                state = last + state[:, :rows]
                head_in[:, :rows, hidden:] = state
            logits = self.raw_logits(head_in[:, :rows])
            if rows != W:
                logits = logits.expand(B, W, V)
                state = state.expand(B, W, hidden)
            log_p_beam, newest, parents, beams, logp = beam_topk_step(
                logits, log_p_beam, beams, want_log_probs=return_log_probs
            )
            state = _gather_beams(state, parents)
            if return_log_probs:
                step_log_probs.append(logp)
                step_parents.append(parents)

        if not return_log_probs:
            return beams, None
        # history[b, w, t] = log-probs of step t under the ancestor of final beam w at step t:
        # compose the parent maps backwards once instead of re-gathering the history every step
        history = torch.empty((B, W, L - 1, V), dtype=torch.float32, device=dev)
        ancestor = torch.arange(W, device=dev).expand(B, W)
        for t in range(L - 2, -1, -1):
            ancestor = torch.gather(step_parents[t], 1, ancestor)
            tree_attention.gather_rows(step_log_probs[t], ancestor.contiguous(), out=history[:, :, t, :])
        return beams, history

    def assert_valid(self) -> None:
        has_proj = hasattr(self, "input_proj")
        assert has_proj == (2 * self.config.hidden_size != self.config.exit_dim)
        assert isinstance(self.lm_head, torch.nn.Sequential)
        assert len(self.lm_head) == self.config.num_draft_layers + 1
