"""tnx_logp_drift_static, the entry point that allocates nothing (its row moments live in an
array built into the library), against tnx_logp_drift with a caller's workspace: identical
results, on two calls in a row with the second input smaller than the first (the array keeps
the first call's rows), and a clear error above the built-in limit."""
import numpy as np
import pytest
import torch

from tunix_amd import _lib as L
from tunix_amd import ops

pytestmark = pytest.mark.gpu


def _case(rng, B, T, gpu):
  a = -rng.gamma(2.0, 1.0, size=(B, T)).astype(np.float32)
  b = (a + rng.normal(0, 0.05, size=(B, T))).astype(np.float32)
  lens = rng.integers(0, T + 1, size=B)
  mask = (np.arange(T)[None, :] < lens[:, None]).astype(np.float32)
  return tuple(torch.from_numpy(v).to(gpu) for v in (a, b, mask))


def test_static_scratch_drift_equals_workspace_drift(gpu):
  rng = np.random.default_rng(31)
  free_before = None
  for B, T in ((512, 300), (37, 64)):   # the second call is smaller and follows the first
    a, b, m = _case(rng, B, T, gpu)
    want = torch.zeros(5, dtype=torch.float32, device=gpu)
    got = torch.full((5,), float("nan"), dtype=torch.float32, device=gpu)
    ops.logp_drift(a, b, m, want)
    torch.cuda.synchronize()
    if free_before is None:
      ops.logp_drift_static(a, b, m, got)   # first call on the device: looks the array up
      torch.cuda.synchronize()
      got.fill_(float("nan"))
    free_before = torch.cuda.mem_get_info()[0]
    ops.logp_drift_static(a, b, m, got)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before   # no device memory taken or returned
    assert torch.equal(got, want), (B, T, got.tolist(), want.tolist())   # same kernels: bit-equal
    assert torch.isfinite(got).all()


def test_static_scratch_drift_rejects_oversize(gpu):
  lim = int(L.lib().tnx_logp_drift_static_max_rows())
  assert lim == 4096
  B = lim + 1
  z = torch.zeros(B, 2, dtype=torch.float32, device=gpu)
  out = torch.zeros(5, dtype=torch.float32, device=gpu)
  with pytest.raises(ValueError, match="built-in scratch"):
    ops.logp_drift_static(z, z, z, out)
  ok = torch.zeros(lim, 2, dtype=torch.float32, device=gpu)   # the limit itself is accepted
  ops.logp_drift_static(ok, ok, torch.ones_like(ok), out)
  torch.cuda.synchronize()
  assert out[0].item() == 0.0 and out[1].item() == 0.0
