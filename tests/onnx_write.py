"""The ONNX writer lives in the package (the benchmark builds its models with it too)."""
from sofie_amd.benchsupport.onnx_write import *  # noqa: F401,F403
from sofie_amd.benchsupport.onnx_write import tensor, attribute, node, value_info, model, write, _vi, _ld, _key, _varint  # noqa: F401
