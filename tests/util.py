"""The counter-based generator and the device-buffer helpers live in the package (the benchmark uses them too)."""
from sofie_amd.benchsupport.synthetic import *  # noqa: F401,F403
from sofie_amd.benchsupport.synthetic import splitmix64, uniform01, normal, int8_sym, int32_range, to_dev, dev_empty, ptr, to_host  # noqa: F401
