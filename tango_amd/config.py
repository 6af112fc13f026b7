"""Process-wide switches of the operator layer (the reference has none; its
behaviour is the default of each)."""
import itertools
import os

# Reproduce the reference's defects where they change numbers:
#   cuda/SPMM.py:56 dequantizes dN with the forward scale sN*sE although dZ was
#   quantized with its own scale.
ref_compat = os.environ.get("TANGO_REF_COMPAT", "0") == "1"

# Rounding used when gradients are quantized in backward passes
# (cuda/QLinear.py:42, cuda/SPMM.py:20,53, cuda/SDDMM.py:26 use half-to-even).
grad_round_mode = os.environ.get("TANGO_GRAD_ROUND", "rne")

# Seed of the counter-based RNG for stochastic rounding; every quantize call
# draws a fresh 2^40-element window of the stream.
seed = int(os.environ.get("TANGO_SEED", "0"))
_calls = itertools.count()


def next_offset():
    return next(_calls) << 40
