"""The reference's NVIDIA search space and hardware descriptors, restated: test data for tests/test_enumeration.py
(the ordered configuration lists in the reference's published tuning logs are the tuner's only known answers).
Nothing here is compiled, launched or imported by the product."""
from . import legacy_space
from .A100 import A100
from .RTX4090 import RTX4090
