"""The CPU chains of the benchmark models live beside the oracle, the models' constants in the package."""
from oracle.chains import int8_mlp_oracle, int8_cnn_oracle  # noqa: F401
from sofie_amd.benchsupport.models import make_int8_cnn  # noqa: F401
