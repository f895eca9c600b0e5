"""Model dimensions of the reference's shipped configurations, as data.

Values are the `gpt_config.init_args` blocks of configs/mvpformer_s_generative.yaml:49-71 and
configs/mvpformer_classification.yaml:49-71 (both carry lora: true, n_positions: 110,
n_channels: 128, layer_norm_epsilon 1e-5, initializer_range 0.02)."""

MVPFORMER_S = dict(n_positions=110, n_channels=128, n_embd=768, n_layer=12, n_head=12,
                   n_head_kv=4, n_inner=1728, global_att=True, activation_function="silu",
                   resid_pdrop=0.1, embd_pdrop=0.1, attn_pdrop=0.1, layer_norm_epsilon=1.0e-05,
                   initializer_range=0.02, scale_attn_weights=True, use_cache=True,
                   scale_attn_by_inverse_layer_idx=False, reorder_and_upcast_attn=False, lora=True)

MVPFORMER_BASE = dict(n_positions=110, n_channels=128, n_embd=2048, n_layer=24, n_head=16,
                      n_head_kv=8, n_inner=5632, global_att=True, activation_function="silu",
                      resid_pdrop=0.1, embd_pdrop=0.1, attn_pdrop=0.1, layer_norm_epsilon=1.0e-05,
                      initializer_range=0.02, scale_attn_weights=True, use_cache=True,
                      scale_attn_by_inverse_layer_idx=False, reorder_and_upcast_attn=False, lora=True)
