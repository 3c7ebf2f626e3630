"""Seeded input generators for the benchmark configurations and small helpers shared by the tests."""
import numpy as np


def rng(seed, stream=0):
    """The build's own counter-based generator: numpy Philox keyed by (seed, stream)."""
    return np.random.Generator(np.random.Philox(key=[seed, stream]))


def grads_f32(seed, P, N, std, step=0):
    return [(rng(seed, 1000 * step + p + 1).standard_normal(N, dtype=np.float32) * np.float32(std)) for p in range(P)]


def weights_f32(seed, N, half_range):
    return rng(seed, 0).uniform(-half_range, half_range, N).astype(np.float32)


def rel_err(a, b):
    """max |a-b| / max(|b|, tiny) elementwise, the form the north-star tolerance is stated in."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    d = np.abs(a - b)
    den = np.maximum(np.abs(b), 1e-30)
    return float(np.max(d / den)) if a.size else 0.0


def ulp_diff_f32(a, b):
    """Largest distance in units in the last place between two fp32 arrays (same-sign finite values)."""
    ia = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    ib = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia)
    ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    return int(np.max(np.abs(ia - ib))) if ia.size else 0


# The reference's own fixture (nccl-overlap/samples/multi-process-adam-scattered.cpp:221-226, :736):
# buffer i holds (i%2+1)*(index%20+1) in both the gradient and the weight, moments start at zero.
def ref_integer_pattern(buff_index, n):
    idx = np.arange(n, dtype=np.int64)
    return ((buff_index % 2 + 1) * (idx % 20 + 1)).astype(np.float32)


# first entries of the reference's buffer-size list (multi-process-adam-scattered.cpp:736), a BERT layer layout
REF_BUFF_SIZES_HEAD = [31260672, 2048, 1048576, 1048576, 1048576, 1048576, 4194304, 4194304]
REF_BUFF_SIZES_TAIL = [1024, 1024, 1024, 1024, 30528, 1024, 1024, 1024]
