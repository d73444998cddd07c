"""Per-tensor absmax e4m3 quantisation on the device: bit-exact against the oracle's e4m3 rounding."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import to_dev_bf16
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,seed,mult", [((4096, 128), 0, 1.0), ((1, 333, 4, 128), 1, 37.0), ((16,), 2, 1e-3)])
def test_quant_matches_oracle_bit_exact(dev, shape, seed, mult):
  x = O.bf16_round(O.normal_bf16(shape, seed) * np.float32(mult))
  x8, sc = ops.quant_e4m3(to_dev_bf16(x, dev))
  ref8, rs = O.quant_e4m3(x)
  sc = sc.cpu().numpy()
  assert sc[1] == np.abs(x).max() and abs(sc[0] - rs) <= 1e-7 * rs
  got = x8.view(torch.float8_e4m3fn).float().cpu().numpy()
  # the kernel multiplies by 448/absmax where the oracle divides by absmax/448: values that land within
  # one f32 ulp of a rounding boundary may fall to the neighbouring code
  mism = got != ref8
  assert mism.mean() <= 1e-4
  assert np.all(np.abs(got - ref8)[mism] <= np.maximum(np.abs(ref8[mism]) / 8, 2.0**-9))


@pytest.mark.parametrize("premul,mult", [(1.0, 1.0), (0.1275174, 1.0), (0.1275174, 37.0), (3.0, 1e-3)])
def test_quant_with_premul_and_power_of_two_scale(dev, premul, mult):
  x = O.bf16_round(O.normal_bf16((2048, 128), 5) * np.float32(mult))
  x8, sc = ops.quant_e4m3(to_dev_bf16(x, dev), premul=premul, pow2_scale=True)
  ref8, rs = O.quant_e4m3(x, premul=premul, pow2_scale=True)
  sc = sc.cpu().numpy()
  m, _ = np.frexp(sc[0])
  assert m == 0.5 and sc[0] == rs                       # a power of two, the oracle's
  assert sc[0] >= np.abs(x).max() * np.float32(premul) / 448 > sc[0] / 2   # the smallest that keeps |x8| <= 448
  got = x8.view(torch.float8_e4m3fn).float().cpu().numpy()
  mism = got != ref8
  assert mism.mean() <= 1e-4
  assert np.all(np.abs(got - ref8)[mism] <= np.maximum(np.abs(ref8[mism]) / 8, 2.0**-9))
  # dequantised values are x * premul to e4m3 precision (3 mantissa bits; denormals below 2^-6 * scale)
  err = np.abs(got * sc[0] - x * np.float32(premul))
  assert np.all(err <= np.maximum(np.abs(x * np.float32(premul)) / 16, sc[0] * 2.0**-10) * 1.001)
