flex_gpu_transformer_name = "flexhip"
