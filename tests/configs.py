"""Tiny configurations of the architecture. A and B differ in every size and option:
layers, width, heads and groups (4/2 vs 3/1), head size, intermediate size, vocabulary,
rope base and scaling (none vs llama3 with all three bands non-empty), the norms' eps,
tied vs untied output matrix. Widths 96 and 3 heads are no powers of two. C has the head
size and group of the 1B model at a small width, so the D=64 kernels run in engine tests."""

from __future__ import annotations

# Wider than the usual 0.02 so that logits are well separated: with near-ties a 1e-7
# difference could flip an argmax (the reference's tests do the same,
# tests/test_llama_exact.py:69-71).
INIT_STD = 0.1

TINY = {
    "A": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=256, hidden_size=64,
              intermediate_size=128, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=2048, tie_word_embeddings=True,
              eos_token_id=2),
    "B": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=512, hidden_size=96,
              intermediate_size=256, num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
              rms_norm_eps=1e-6, rope_theta=500000.0,
              rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                original_max_position_embeddings=64),
              max_position_embeddings=4096, tie_word_embeddings=False, eos_token_id=[1, 2]),
    "C": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1000, hidden_size=256,
              intermediate_size=688, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2, head_dim=64,
              rms_norm_eps=1e-5, rope_theta=500000.0,
              rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                original_max_position_embeddings=128),
              max_position_embeddings=4096, tie_word_embeddings=True),
}

# Relative to max|logit| of the compared rows.
TOL_F32 = 1e-4      # the reference's bar for its exact tier (tests/test_llama_exact.py:42)
# bfloat16 keeps 8 bits: 2^-8 per rounding, a few tens of roundings deep. How far that moves a
# row of logits is a property of the model, so a row is held to BF16_ROW_FACTOR x the worst row
# of a plain bfloat16 run of the same model over the same or as many tokens (conftest's
# bf16_row_bar and checks.plain_bf16_bars; the worst rows of plain models of random
# configurations lie between 2.5e-2 and 7.5e-2), and the mean to that run's mean.
BF16_ROW_FACTOR = 1.5
