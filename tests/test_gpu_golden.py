"""The reference's own attention vectors through the HIP kernels.

tests/golden/sdpa_golden.json holds the six cases of the reference's tests/attention_golden.rs
(inputs and expected outputs as literals; used there by tests/nn_attention.rs:33-56).  Their head
sizes are 4 and 8; the kernels take 64 or 128, so q, k and v are zero-padded along the channel axis
(zero channels add nothing to q.k and give zero output channels) and the scale is passed as
1/sqrt(original head size).  Additive and boolean masks become the kernels' dense [n, n] mask
(boolean: 0 where allowed, -inf where not), the causal case uses the flag, GQA the kv-head count.
Tolerance: the reference's own measure, |got - want| <= tol * max(|want|, 1) (tests/nn_attention.rs:11-24),
with its tol = 1e-5 for fp32 and tol = 2e-2 for bf16 and int8 against these fp32 results (the vectors
reach 19, where a bf16-stored output alone is off by up to 2^-9 * 19 = 0.04).
"""
import json
import os

import numpy as np
import pytest

from autorust_amd.device import BF16, F32
from gpu_util import run_flash, run_sage

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "sdpa_golden.json")


def _cases():
    with open(GOLDEN) as fh:
        return json.load(fh)["cases"]


def _load(c, D):
    def arr(key):
        a = np.array(c[key], np.float32).reshape(c[key + "_shape"])
        return a[:, None] if a.ndim == 3 else a          # 3-D inputs are [batch, n, d]
    q, k, v, want = arr("q"), arr("k"), arr("v"), arr("out")
    d0 = q.shape[-1]
    pad = lambda t: np.ascontiguousarray(np.pad(t, [(0, 0)] * 3 + [(0, D - d0)]))
    mask = None
    if c["mask_shape"]:
        m = np.array(c["mask"], np.float32).reshape(c["mask_shape"])
        if c["mask_bool"]:
            m = np.where(m != 0, np.float32(0), np.float32(-np.inf))
        assert m.shape[0] == 1                            # broadcast over batch: one [n, n] mask
        mask = np.ascontiguousarray(m.reshape(m.shape[-2], m.shape[-1]))
    return pad(q), pad(k), pad(v), mask, want, d0


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
def test_reference_vectors_fp32_exact_kernel(dev, case, D):
    q, k, v, mask, want, d0 = _load(case, D)
    got = run_flash(dev, q, k, v, F32, mask=mask, causal=case["is_causal"], scale=1.0 / np.sqrt(np.float32(d0)))
    assert not got[..., d0:].any()
    assert np.all(np.abs(got[..., :d0] - want) <= 1e-5 * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
def test_reference_vectors_bf16_kernel(dev, case, D):
    q, k, v, mask, want, d0 = _load(case, D)
    got = run_flash(dev, q, k, v, BF16, mask=mask, causal=case["is_causal"], scale=1.0 / np.sqrt(np.float32(d0)))
    assert not got[..., d0:].any()
    assert np.all(np.abs(got[..., :d0] - want) <= 2e-2 * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
def test_reference_vectors_int8_kernel(dev, case):
    """The quantised path on the same vectors with the reference's own granularity (one scale per
    row, no smoothing): int8 costs about 1e-2 on inputs of this size."""
    q, k, v, mask, want, d0 = _load(case, 64)
    res = run_sage(dev, q, k, v, 1, 1, smooth=False, mask=mask, causal=case["is_causal"],
                   scale=1.0 / np.sqrt(np.float32(d0)))
    assert np.all(np.abs(res["out"][..., :d0] - want) <= 2e-2 * np.maximum(np.abs(want), 1.0))
