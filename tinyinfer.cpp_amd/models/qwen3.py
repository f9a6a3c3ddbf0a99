"""The Qwen3 dense decoder: its typed configuration and its `ModelSpec` come from
the host library (`build_qwen3_spec`, config/config.cpp; layer order and
formulas: /root/reference/src/inference.cu:28-72), under the names
"Qwen3ForCausalLM" and "qwen3".  `registry.config_and_spec` finds it there."""
