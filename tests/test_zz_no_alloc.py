"""mesh_moe_top2_gating_static_scratch (the entry point that takes no workspace
and allocates nothing) against mesh_moe_top2_gating, through the C ABI.

Both run the same kernels, so every output must agree bit for bit; the routing
is also compared with the CPU oracle.  Two calls in a row share the library's
built-in scratch array, the second on a smaller input, so stale contents of the
first call would show.
"""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
  from mesh_amd import moe_hip
  moe_hip.load_library()
  return moe_hip


def _empty_routing(hip, g, s, e, fill_byte):
  """Caller-owned outputs, pre-filled so that an entry the call does not write
  would show."""
  def buf(shape, dtype):
    t = torch.empty(shape, dtype=dtype, device="cuda")
    t.view(torch.uint8).fill_(fill_byte)
    return t
  return hip.Routing(buf((g, s, 2), torch.int32), buf((g, s, 2), torch.int32),
                     buf((g, s, 2), torch.float32), buf((g, s, 2), torch.uint8),
                     buf((g, e), torch.int32), buf((1,), torch.float32), 0, e)


def _assert_bitwise_equal(got, want):
  for name in ("idx", "pos", "gate", "kept", "fill", "loss"):
    a, b = getattr(got, name), getattr(want, name)
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name


# (G, S, E, C, options): a large call first, then a smaller one on the same
# scratch array; the second also exercises the second-place loss, whose
# partial sums use the half of the scratch the first call left untouched.
CALLS = [
    (16, 2048, 64, 32, dict()),
    (3, 300, 24, 9, dict(use_second_place_loss=True, policy="threshold",
                         threshold=0.3, num_microbatches=2)),
]


def test_static_scratch_matches_workspace_entry(hip):
  rng = np.random.default_rng(2024)
  got, alive = None, []   # nothing is released between the allocator readings
  for call, (g, s, e, c, opts) in enumerate(CALLS):
    logits = H.safe_logits(rng, g, s, e, scale=1.5)
    lg = torch.from_numpy(logits).cuda()
    imp = None
    if call == 1:
      imp_np = rng.choice(np.array([0.0, 0.5, 1.0], np.float32), size=(g, s),
                          p=[0.1, 0.2, 0.7])
      imp = torch.from_numpy(imp_np).cuda()
      opts = dict(opts, importance=imp)
    want = hip.top2_gating(lg, c, **opts)
    out = _empty_routing(hip, g, s, e, 0xA5 if call == 0 else 0x5A)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    alive.append(got)
    got = hip.top2_gating_static_scratch(lg, c, out, **opts)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    _assert_bitwise_equal(got, want)
    okw = {k: v for k, v in opts.items() if k != "importance"}
    oracle = O.top_2_gating(logits, c, importance=None if imp is None else imp_np,
                            **okw)
    got_np = H.routing_to_np(got)
    H.assert_routing_equal(got_np, oracle)
    np.testing.assert_allclose(got_np["loss"], oracle["loss"], rtol=2e-5)


def test_static_scratch_rejects_sizes_beyond_its_array(hip):
  lib = hip.load_library()
  g, s, e = 512, 16384, 512          # needs far more than the built-in array
  assert lib.mesh_moe_gating_workspace_bytes(g, s, e) > hip.STATIC_SCRATCH_BYTES
  one = torch.zeros((1,), device="cuda")
  rc = lib.mesh_moe_top2_gating_static_scratch(
      one.data_ptr(), None, 0, 0, None, g, s, e, 4, 0, 0.2, 0, 1,
      one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(),
      one.data_ptr(), one.data_ptr(), None)
  assert rc == -2
  assert b"scratch" in lib.mesh_moe_last_error()
