"""The tiny configurations that the tests run.  A and B differ in every size and option:
layers, hidden size, head counts and groups, head_dim (A: heads x head_dim == hidden,
B: != hidden), intermediate size, vocabulary, rope_theta, the norms' eps, tied or untied
head, positions.  C has sizes that are no power of two anywhere.  D has the sizes that the
decode kernels with tiled weights and folded norms need (inner sizes in multiples of 128, outer
ones of 16), so that steps of few rows take those kernels in bfloat16."""

TINY_A = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=2,
              hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128,
              vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              max_position_embeddings=128, bos_token_id=1, eos_token_id=2)

TINY_B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=3,
              hidden_size=96, num_attention_heads=8, num_key_value_heads=2, head_dim=32, intermediate_size=160,
              vocab_size=384, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
              max_position_embeddings=256, bos_token_id=0, eos_token_id=5)

TINY_C = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=2,
              hidden_size=88, num_attention_heads=6, num_key_value_heads=3, head_dim=48, intermediate_size=200,
              vocab_size=331, rope_theta=50000.0, rms_norm_eps=3e-6, tie_word_embeddings=False,
              max_position_embeddings=640, bos_token_id=0, eos_token_id=7)

TINY_D = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=3,
              hidden_size=128, num_attention_heads=4, num_key_value_heads=1, head_dim=64, intermediate_size=384,
              vocab_size=400, rope_theta=20000.0, rms_norm_eps=2e-6, tie_word_embeddings=True,
              max_position_embeddings=320, bos_token_id=0, eos_token_id=3)

#: the head size and group shape of the large models (128-wide heads, several query heads per kv head), small otherwise
TINY_E = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=2,
              hidden_size=256, num_attention_heads=8, num_key_value_heads=2, head_dim=128, intermediate_size=640,
              vocab_size=592, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
              max_position_embeddings=448, bos_token_id=0, eos_token_id=4)

#: init that makes attention and logits informative: matrices N(0, std), norms 1 + N(0, 0.1)
INIT = dict(matrix_std=0.08, norm_std=0.1)
