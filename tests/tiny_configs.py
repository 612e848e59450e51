"""Tiny LFM2 configurations for tests. A and B differ in every size and
option; C adds a sliding window on some attention layers (a second cache
group) and float32-stored tensors.

`max_position_embeddings` of A and B is 1024 and 2048, eight times what models
of this size would state (128 and 256), because the tests run sequences of 150
to 330 tokens through them (portions over several pages, long decoding, mixed
schedules that use pages again) and the engine refuses a request that would
pass the model's positions. Nothing in the computation reads that number."""

TINY_A = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2",
    vocab_size=256, hidden_size=64, num_hidden_layers=4,
    layer_types=["conv", "full_attention", "conv", "full_attention"],
    num_attention_heads=4, num_key_value_heads=2,
    block_auto_adjust_ff_dim=False, block_ff_dim=192,
    conv_L_cache=3, conv_bias=False, rope_theta=10000.0, tie_embedding=True,
    norm_eps=1e-5, max_position_embeddings=1024,
)

TINY_B = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2",
    vocab_size=384, hidden_size=96, num_hidden_layers=6,
    layer_types=["conv", "conv", "full_attention", "conv", "full_attention", "full_attention"],
    num_attention_heads=3, num_key_value_heads=1,
    block_auto_adjust_ff_dim=True, block_ff_dim=480, block_multiple_of=64, block_ffn_dim_multiplier=1.0,
    conv_L_cache=4, conv_bias=True, rope_theta=1000000.0, tie_embedding=False,
    norm_eps=1e-6, max_position_embeddings=2048,
)

TINY_C = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2",
    vocab_size=200, hidden_size=160, num_hidden_layers=5,
    layer_types=["sliding_attention", "conv", "full_attention", "sliding_attention", "conv"],
    num_attention_heads=10, num_key_value_heads=5,
    block_auto_adjust_ff_dim=False, block_ff_dim=172,
    conv_L_cache=2, conv_bias=False, rope_theta=50000.0, tie_embedding=True,
    norm_eps=1e-4, max_position_embeddings=1024, sliding_window=24,
)

CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2)}
# tensors of C kept in float32 in the file: norms and one layer's matrices
C_KEEP_F32 = ("norm", "layers.1.conv.in_proj", "layers.2.self_attn.q_proj")
