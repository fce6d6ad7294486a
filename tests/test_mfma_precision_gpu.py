"""What the MI355X matrix unit does to the sums, measured live and held against oracle/mfma_model.py.

1. The exponent-ladder cases of tests/golden/mfma_ladder.json are re-run through several kernel families: the hardware
   has to return the recorded bits (so the fixture, which pins the model on GPU-less machines, stays true).
2. Whole GEMMs on quantised random data at fp32 output are compared with the model: the kernels may differ from it by
   the order of a few fp32 additions (1e-6 of the result's rms), not by a truncation step (1e-4).  This is the parity
   check at the strict floor: relative error against the model with |ref| floored at 1e-3 rms.
3. The distance between the model and the exact oracle is the documented cost of the hardware's truncation.
"""
import json
import os
import sys

import numpy as np
import pytest
import torch

import helpers
from oracle import fp8_block_gemm as orc
from oracle import mfma_model

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
if GOLDEN not in sys.path:
    sys.path.insert(0, GOLDEN)


@pytest.fixture(scope='module')
def dev():
    from dlblas_amd import _lib
    _lib.load()
    return torch.device('cuda:0')


def _gemm(dev, a_q, a_s, b_q, b_s, dtype, variant=None):
    from dlblas_amd import _lib
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        _lib.force_variant(variant)
        out = fp8_gemm(a_q.to(dev), b_q.to(dev), torch.as_tensor(a_s).to(dev), torch.as_tensor(b_s).to(dev))
        torch.cuda.synchronize()
    finally:
        _lib.force_variant(None)
        torch.set_default_dtype(prev)
    return out.cpu()


@pytest.mark.parametrize('variant', ['skinny16', 'skinny128', 'tile128x128', 'pipe256x256', 'pipe128x256w8', 'pipe128x128', 'pipe256mix'])
def test_ladder_cases_give_the_recorded_bits(dev, variant):
    import make_mfma_ladder
    print(f'case mfma ladder variant={variant}', flush=True)
    with open(os.path.join(GOLDEN, 'mfma_ladder.json')) as fh:
        cases = json.load(fh)['cases']
    if variant == 'skinny16':
        cases = cases[:16]  # this variant takes at most 16 rows
        a_q, b_q = make_mfma_ladder.operands(cases)
        a_q = a_q[:16]
    else:
        a_q, b_q = make_mfma_ladder.operands(cases)
    out = _gemm(dev, a_q, np.ones((a_q.shape[0], 1), np.float32), b_q, np.ones((b_q.shape[0] // 128, 1), np.float32),
                torch.float32, variant)
    got = out.diagonal()[:len(cases)].double().tolist()
    for c, v in zip(cases, got):
        assert v == c['out'], f"{variant}: {c['name']}: {v!r} != recorded {c['out']!r}"


MODEL_SHAPES = [
    (64, 512, 1024, None),            # the reference's CPU-runnable configuration
    (16, 384, 2048, None),            # decode kernel
    (128, 256, 1024, 'skinny128'),
    (200, 392, 1024, 'tile128x128'),  # ragged tiles, register-staged kernel
    (256, 512, 1024, 'pipe256x256'),  # the prefill kernel
    (256, 576, 768, 'pipe256mix'),    # ... with the narrow-tile region
    (128, 256, 512, 'pipe128x128'),   # register-double-buffered ring kernel
]


@pytest.mark.parametrize('M,N,K,variant', MODEL_SHAPES)
def test_kernels_match_the_model_at_the_strict_floor(dev, M, N, K, variant):
    print(f'case model parity M={M} N={N} K={K} variant={variant}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=41)
    model = mfma_model.gemm_model(a_q, a_s.numpy(), b_q, b_s.numpy())
    model_t = torch.from_numpy(model)
    rms = float(np.sqrt((model.astype(np.float64)**2).mean()))
    out32 = _gemm(dev, a_q, a_s, b_q, b_s, torch.float32, variant)
    worst = float((out32.double() - model_t.double()).abs().max())
    strict = orc.max_rel_err(out32, model_t, 1e-3)
    print(f'  fp32 out vs model: max |diff| = {worst / rms:.2e} rms, relative error at the 1e-3 rms floor = {strict:.2e}', flush=True)
    assert worst <= 5e-6 * rms, f'kernel and model differ by {worst / rms:.2e} rms: more than summation order explains'
    assert strict <= 1e-2
    out16 = _gemm(dev, a_q, a_s, b_q, b_s, torch.bfloat16, variant)
    allowed = 2.0**-8 * model_t.double().abs() + 5e-6 * rms
    assert bool(((out16.double() - model_t.double()).abs() <= allowed).all()), 'bf16 output is not the rounded model value'
    # the stated bar of the north star, at the survey's floor, against the model of what the hardware computes
    assert orc.max_rel_err(out16.float(), model_t, 1e-3) <= 1e-2
    # what the truncation costs against exact arithmetic (reported; bounded by the parity floor of helpers.tolerance_check)
    exact = orc.dequant_ref(a_q, a_s, b_q, b_s)
    gap = float((model_t.double() - exact.double()).abs().max())
    print(f'  model vs exact oracle: max |diff| = {gap / rms:.2e} rms', flush=True)
    assert gap <= 3e-4 * rms
