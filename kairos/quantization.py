from kairos_amd.weight_prep import quantize_tensor_int8, kairos_quantize_tensor_int4  # noqa: F401
