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

# spmm_u_mul_e with a scale handed in (the edge softmax's kernel finds it): round the fp32 edge values inside the
# aggregation as they are loaded (no int8 copy, no quantize launch) instead of in a pass of their own.
edge_values_on_load = os.environ.get("TANGO_EDGE_ON_LOAD", "0") == "1"

# gat_edge_attention: form the logits q(el)[src] + q(er)[dst] inside the softmax kernel instead of storing them with
# the element-wise SDDMM first.  Same values; measured slower on the benchmark graphs (the two dependent gathers
# per slot lengthen the softmax kernel's latency chain by more than the stored tensor costs), hence off.
attention_logits_on_the_fly = os.environ.get("TANGO_ATTN_ON_THE_FLY", "0") == "1"

# spmm_copy_u on dense graphs: let the aggregation's epilogue return the scale of its output (forward: to the next
# layer's GEMM; backward: to the quantizer of the gradient it produces) instead of a pass over that output.  Same
# values.  Measured on the 114.8 M-edge benchmark epoch: the passes it removes take 100 us and the reduction over
# the per-row maxima adds 17, but the gather launches that carry the epilogue take 130 us longer in all (57 us each
# at 256 columns): 5.22 against 5.17 ms per epoch, hence off.  The epilogue needs 65 instead of 64 VGPRs (seven
# instead of eight waves per SIMD); held at 64 by a launch bound (two dwords spilled in the epilogue) it costs the same.
scale_from_aggregation = os.environ.get("TANGO_SCALE_FROM_AGGREGATION", "0") == "1"

# Seed of the counter-based RNG for stochastic rounding; every quantize call
# draws a fresh 2^40-element window of the stream.
seed = int(os.environ.get("TANGO_SEED", "0"))
WINDOW = 1 << 40
_calls = itertools.count()
_counters = {}


def next_offset():
    """Host-side position in the stream (a Python counter): for callers that pass ``offset`` as a number."""
    return next(_calls) * WINDOW


def device_offset(device):
    """The position in the stream as one int64 word in ``device``'s memory.  The quantize kernels add it to their
    offset when they start and a one-thread kernel on the same stream advances it (see ``stochastic_args`` for
    when), so the position moves with the work itself: a captured graph that is replayed draws a fresh window
    per replay, where a host-side counter would be frozen into the captured launch."""
    import torch
    key = torch.device(device)
    if key.index is None and key.type == "cuda":
        key = torch.device("cuda", torch.cuda.current_device())
    c = _counters.get(key)
    if c is None:
        c = _counters[key] = torch.zeros(1, dtype=torch.int64, device=key)
    return c


def reset_offsets():
    """Back to the start of the stream (tests that compare with a host-side replay of the same draws)."""
    global _calls
    _calls = itertools.count()
    _pending.clear()
    for c in _counters.values():
        c.zero_()


# Calls since a device's counter last moved.  Outside a stream capture the position of a call is
# (device counter) + (pending calls) * WINDOW with the second term passed by value, and the counter moves once per
# BATCH calls: one one-thread launch per BATCH quantize launches instead of one each.  A call recorded into a HIP
# graph draws from a part of the stream of its own (CAPTURE_BASE set in its offset) at the device counter's value
# when the graph runs, and moves the counter by one window itself, so that every replay draws fresh windows; the
# host-side count of pending eager calls is left alone (a capture only records kernels: the counter does not move
# at capture time, and eager calls made afterwards must not start again at the counter's own value).
BATCH = 64
CAPTURE_BASE = 1 << 62
_pending = {}


def stochastic_args(device):
    """Keyword arguments of a stochastically rounding quantize call."""
    import torch
    c = device_offset(device)
    if torch.cuda.is_current_stream_capturing():
        return {"seed": seed, "offset": (CAPTURE_BASE, c), "advance": WINDOW}
    k = _pending.get(c, 0)
    if k + 1 >= BATCH:
        _pending[c] = 0
        return {"seed": seed, "offset": (k * WINDOW, c), "advance": (k + 1) * WINDOW}
    _pending[c] = k + 1
    return {"seed": seed, "offset": (k * WINDOW, c), "advance": 0}
