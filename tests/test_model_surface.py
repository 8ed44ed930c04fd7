"""The model classes as the reference's own model tests use them: the drafter registers with
transformers' Auto classes and survives a save / load round trip (modeling_drafter_test.py:20-33);
the Llama wrapper gives the logits of transformers' LlamaForCausalLM on the same checkpoint
(modeling_llama_test.py:15-50, :68-100: same prompt, same tolerances)."""
import os
import sys
import tempfile

import pytest
import torch
import transformers

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ml-recurrent-drafter_amd"))
import recurrent_drafting_amd as rd  # noqa: E402


def test_register_drafter_auto_models_and_reload():
    rd.modeling_drafter.register_auto_models()
    cfg = rd.configuration_drafter.DrafterConfig(vocab_size=128, hidden_size=16, exit_dim=24, num_draft_layers=1)
    drafter = rd.modeling_drafter.Drafter(cfg)
    with tempfile.TemporaryDirectory() as d:
        drafter.save_pretrained(d)
        again = transformers.AutoModel.from_pretrained(d)
    assert isinstance(again, rd.modeling_drafter.Drafter)
    again.assert_valid()
    assert hasattr(again, "input_proj")  # 2 * 16 != 24
    for (ka, va), (kb, vb) in zip(sorted(drafter.state_dict().items()), sorted(again.state_dict().items())):
        assert ka == kb and torch.equal(va, vb)


def _tiny_llama_config(n_kv_heads):
    from transformers.models.llama.configuration_llama import LlamaConfig

    return LlamaConfig(
        bos_token_id=1, eos_token_id=2, hidden_act="silu", hidden_size=32, initializer_range=0.02,
        intermediate_size=20, max_position_embeddings=4096, num_attention_heads=4, num_hidden_layers=2,
        num_key_value_heads=n_kv_heads, pad_token_id=0, rms_norm_eps=1e-05, tie_word_embeddings=False,
        use_cache=True, vocab_size=11, attention_bias=False, mlp_bias=False,
    )


@pytest.mark.gpu
@pytest.mark.parametrize("n_kv_heads", [4, 2])
def test_llama_logits_equal_transformers_on_one_checkpoint(n_kv_heads):
    """A checkpoint written by this package's model loads into transformers' Llama and back, and
    both give the same logits on the reference's prompt (which starts with the pad id: a
    left-padded row)."""
    torch.manual_seed(3)
    cfg = _tiny_llama_config(n_kv_heads)
    mine = rd.modeling_llama.LlamaForCausalLM(cfg)
    with tempfile.TemporaryDirectory() as d:
        mine.save_pretrained(d)
        as_f32 = {"dtype" if int(transformers.__version__.split(".")[0]) >= 5 else "torch_dtype": torch.float32}
        theirs = transformers.AutoModelForCausalLM.from_pretrained(d, **as_f32)
        mine = rd.modeling_llama.LlamaForCausalLM.from_pretrained(d, **as_f32)
    dev = torch.device("cuda")
    theirs, mine = theirs.to(dev).eval(), mine.to(dev).eval()
    input_ids = torch.tensor([[0, 1, 2, 3, 4, 5, 6], [0, 0, 7, 8, 9, 10, 3]], device=dev)
    pad = 0
    B, S = input_ids.shape
    with torch.inference_mode():
        logits_theirs = theirs(input_ids, attention_mask=input_ids != pad).logits
        cache = rd.kv_cache.Cache(B, S + 1, cfg.num_hidden_layers, cfg.num_key_value_heads,
                                  cfg.hidden_size // cfg.num_attention_heads, torch.float32, dev)
        mask = rd.attention.causal_mask(input_ids != pad, S, dev)
        # positions as the reference's parity check gives them: 0..S-1 in every row
        position_ids = torch.arange(S, device=dev).expand(B, S)
        logits_mine = mine(input_ids, past_key_values=cache.sliced, attention_mask=mask,
                           position_ids=position_ids).logits
    # row 0 is the reference's own case (one leading pad, a token that nobody else attends to);
    # row 1 has two.  The pad positions themselves attend to nothing and are not compared.
    torch.testing.assert_close(logits_theirs[0, 1:], logits_mine[0, 1:], atol=1e-4, rtol=1e-2)
    torch.testing.assert_close(logits_theirs[1, 2:], logits_mine[1, 2:], atol=1e-4, rtol=1e-2)
    assert torch.isfinite(logits_mine).all()
    # the second forward of the wrapper, one more token on the cache, against transformers' full pass
    with torch.inference_mode():
        more = torch.tensor([[4], [5]], device=dev)
        ids2 = torch.cat((input_ids, more), 1)
        logits_theirs2 = theirs(ids2, attention_mask=ids2 != pad).logits[:, -1]
        mask2 = rd.attention.causal_mask(ids2 != pad, 1, dev)
        logits_mine2 = mine(more, past_key_values=cache.sliced, attention_mask=mask2,
                            position_ids=torch.full((B, 1), S, device=dev)).logits[:, -1]
    torch.testing.assert_close(logits_theirs2, logits_mine2, atol=1e-4, rtol=1e-2)
    # the forward has fused the projection weights into shared buffers; unfused, the model saves
    # again and the checkpoint still loads into transformers with the same values
    rd.modeling_llama.unfuse_weights(mine)
    with tempfile.TemporaryDirectory() as d:
        mine.save_pretrained(d)
        again = transformers.AutoModelForCausalLM.from_pretrained(d, **as_f32)
    for k, v in theirs.state_dict().items():
        assert torch.equal(v.cpu(), again.state_dict()[k].cpu()), k
