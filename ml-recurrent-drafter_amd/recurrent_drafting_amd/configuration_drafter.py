"""Configuration of the recurrent drafter head (same fields and model_type as the reference's
recurrent_drafting/configuration_drafter.py, so saved drafters load unchanged)."""

import transformers


class DrafterConfig(transformers.PretrainedConfig):
    model_type = "recurrent_drafting_drafter"

    def __init__(self, vocab_size=-1, hidden_size=-1, exit_dim=-1, num_draft_layers=-1,
                 num_lookback_tokens=-1, rnn=False, **kwargs):
        super().__init__(**kwargs)
        self.vocab_size = vocab_size  # output vocabulary of the drafter's lm_head
        self.hidden_size = hidden_size  # == hidden size of the base LLM
        self.exit_dim = exit_dim  # width of the residual blocks (2*hidden_size: no input_proj)
        self.num_draft_layers = num_draft_layers  # residual blocks in front of the vocabulary matrix
        self.num_lookback_tokens = num_lookback_tokens
        self.rnn = rnn  # recurrent state update with rnn_w / rnn_u
