"""Shared helpers of the GPU parity tests: seeded inputs as numpy arrays, copies to and from
the device, and the comparison metrics (the reference's calc_diff among them)."""
import numpy as np
import torch

from oracle import oracle as zo


def rng(seed):
    return np.random.default_rng(seed)


def dev(a, dtype=None):
    """numpy -> cuda tensor. uint16 arrays carry bf16/fp16 bit patterns (pass dtype), uint8 may carry e4m3."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if a.dtype == np.uint16:
        t = t.view(torch.int16).view(dtype or torch.bfloat16)
    elif dtype is not None and a.dtype == np.uint8:
        t = t.view(dtype)
    return t.cuda()


def host(t):
    """cuda tensor -> numpy; 16-bit floats come back as uint16 bit patterns, e4m3 as uint8."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    return t.numpy()


def bf16_normal(shape, seed, scale=1.0):
    return zo.f32_to_bf16((rng(seed).standard_normal(shape) * scale).astype(np.float32))


def distinct_topk(T, E, K, seed, zipf=None):
    """K distinct experts per token; uniform, or Zipf(s)-skewed popularity over a fixed random permutation."""
    g = rng(seed)
    if zipf is None:
        return np.stack([g.permutation(E)[:K] for _ in range(T)]).astype(np.int64)
    p = 1.0 / np.arange(1, E + 1) ** zipf
    p = p[g.permutation(E)]
    p /= p.sum()
    return np.stack([g.choice(E, size=K, replace=False, p=p) for _ in range(T)]).astype(np.int64)


def calc_diff(x, y):
    """Reference metric, app/zbal/test/python/deepep/utils.py:129-133."""
    x = x.astype(np.float64) + 1
    y = y.astype(np.float64) + 1
    return 1 - 2 * (x * y).sum() / (x * x + y * y).sum()


def max_rel_err(got, want):
    """max |got - want| relative to the largest reference magnitude."""
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def elem_rel_err(got, want, floor_frac=1.0 / 64):
    """max |got - want| / |want| over the elements whose reference magnitude is at least floor_frac of the largest
    one: the element-wise companion of max_rel_err (which divides every difference by the largest magnitude)."""
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    big = np.abs(want) >= floor_frac * max(np.abs(want).max(), 1e-30)
    return float((np.abs(got - want)[big] / np.abs(want)[big]).max()) if big.any() else 0.0


FP8_GEMM_ELEM_TOL = 1.6e-2      # two bf16 roundings of slack on a single GEMM output element
# A whole fp8 layer, element by element (elements of at least 1/64 of the largest magnitude): the worst one, and how
# many may be off by more than FP8_LAYER_ELEM_COMMON. One e4m3 code of the re-quantised intermediate is a 2^-4 step.
FP8_LAYER_ELEM_TOL = 0.5
FP8_LAYER_ELEM_COMMON = 5e-2
FP8_LAYER_ELEM_COMMON_FRACTION = 1e-2


def assert_fp8_close(got, want, what="", elem_tol=None, layer=False):
    """The bar for the block-scaled fp8 path: max error relative to the largest magnitude below 2e-2 (the stated
    tolerance). elem_tol adds an element-wise bound over the elements of appreciable size (>= 1/64 of the largest):
    used for single GEMMs, where the only difference from the oracle is the summation order inside a 128-deep
    block. A whole layer is not held to it: the re-quantisation between the GEMMs can move an intermediate to the
    neighbouring e4m3 code (a 2^-4 step), and the weighted combine cancels, so single small outputs may differ by
    tens of per cent while the layer agrees to 1e-4 in the reference's calc_diff; with layer=True it is held to
    the looser FP8_LAYER_* bounds instead (worst element, and how many may be off by more than a few per cent).
    Returns the figures."""
    g, w = got.astype(np.float64), want.astype(np.float64)
    e_max, e_elem = max_rel_err(g, w), elem_rel_err(g, w)
    assert e_max < 2e-2, "%s: max error relative to the largest magnitude %.3g" % (what, e_max)
    if elem_tol is not None:
        assert e_elem < elem_tol, "%s: element-wise relative error %.3g" % (what, e_elem)
    if layer:
        big = np.abs(w) >= max(np.abs(w).max(), 1e-30) / 64
        rel = np.abs(g - w)[big] / np.abs(w)[big]
        frac = float((rel > FP8_LAYER_ELEM_COMMON).mean()) if rel.size else 0.0
        assert e_elem < FP8_LAYER_ELEM_TOL, "%s: element-wise relative error %.3g" % (what, e_elem)
        assert frac < FP8_LAYER_ELEM_COMMON_FRACTION, "%s: %.3g of the elements are off by more than %g" % (what, frac, FP8_LAYER_ELEM_COMMON)
        return e_max, e_elem, frac
    return e_max, e_elem
