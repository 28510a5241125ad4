"""Shared test utilities: seeded rank buffers and torch<->oracle carriers."""
import numpy as np
import torch

from oracle import oracle as O

SEED = 1234

TORCH_TO_CODE = {
    torch.uint8: O.U8, torch.int8: O.I8, torch.int16: O.I16, torch.int32: O.I32,
    torch.int64: O.I64, torch.float16: O.F16, torch.float32: O.F32, torch.float64: O.F64,
    torch.bfloat16: O.BF16,
}
ALL_DTYPES = list(TORCH_TO_CODE)
FLOAT_DTYPES = [torch.float16, torch.bfloat16, torch.float32, torch.float64]
INT_DTYPES = [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64]


def rank_generator(seed, rank):
    """One generator per (seed, rank)."""
    return torch.Generator(device="cpu").manual_seed(seed * 1_000_003 + rank)


def rank_buffer(count, dtype, rank, seed=SEED, dist="normal", scale=0.02):
    """Seeded values: fp32 sample -> scale -> round to the storage dtype (floats);
    uniform integers over a range that exercises wrap-around (ints)."""
    g = rank_generator(seed, rank)
    if dtype.is_floating_point:
        if dist == "normal":
            x = torch.randn(count, generator=g, dtype=torch.float32) * scale
        else:  # uniform[-1, 1)
            x = torch.rand(count, generator=g, dtype=torch.float32) * 2.0 - 1.0
        return x.to(dtype)
    info = torch.iinfo(dtype)
    lo, hi = max(info.min, -(2 ** 62)), min(info.max, 2 ** 62)
    return torch.randint(lo, hi, (count,), generator=g, dtype=torch.int64).to(dtype)


def to_carrier(t):
    """torch CPU tensor -> numpy array in the oracle's carrier dtype (bit patterns for 16-bit floats)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16).reshape(-1)
    return t.numpy().reshape(-1)


def bits(t):
    """Bit pattern of a tensor as an unsigned numpy array (for exact comparisons)."""
    t = t.detach().cpu().contiguous()
    width = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[t.element_size()]
    itype = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.view(itype).numpy().view(width).reshape(-1)


def assert_bits_equal(actual_bits, expected_bits, what=""):
    actual_bits = np.asarray(actual_bits).reshape(-1)
    expected_bits = np.asarray(expected_bits).reshape(-1)
    assert actual_bits.shape == expected_bits.shape, (what, actual_bits.shape, expected_bits.shape)
    bad = np.nonzero(actual_bits != expected_bits)[0]
    if bad.size:
        i = int(bad[0])
        raise AssertionError("%s: %d of %d elements differ; first at %d: got 0x%x want 0x%x" % (
            what, bad.size, actual_bits.size, i, int(actual_bits[i]), int(expected_bits[i])))


def oracle_reduce_bits(cpu_tensors, op=O.SUM):
    code = TORCH_TO_CODE[cpu_tensors[0].dtype]
    out = O.reduce([to_carrier(t) for t in cpu_tensors], code, op)
    width = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[out.dtype.itemsize]
    return out.view(width)
