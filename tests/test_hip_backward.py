"""GPU parity of the backward C-ABI entry points against the CPU oracle's
backward (itself pinned by central differences in tests/test_oracle.py)."""

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


def _hp(**kw):
  base = dict(moe_second_policy_train="all", moe_second_policy_eval="all",
              moe_switch_policy_train="argmax", moe_switch_policy_eval="argmax")
  base.update(kw)
  return O.default_hparams(**base)


def run_backward(hip, x, w, hp, act_dtype, d_out, d_loss, nonpad, mb):
  """The forward and backward call sequence of one v1 layer through the C ABI
  (what MoEV1Operation and its gradient do), on [G, S, M] tokens."""
  g, s, m = x.shape
  e, hdim = hp.moe_num_experts, hp.moe_hidden_size
  n = w["wo"].shape[-1]
  c = O.expert_capacity(s, hp.moe_capacity_factor_train, e,
                        hp.moe_min_expert_capacity)
  xg = H.to_gpu(x, act_dtype)
  wg, wi, wo = (H.to_gpu(O.cast_act(w[k], act_dtype), act_dtype)
                for k in ("w_gate", "wi", "wo"))
  imp = None if nonpad is None else H.to_gpu(nonpad, act_dtype)
  wg_p = hip.pack_weights(wg.reshape(1, m, e), wg.dtype)
  wi_p, wo_p = hip.pack_weights(wi, wi.dtype), hip.pack_weights(wo, wo.dtype)
  logits = hip.router_logits(xg.reshape(1, g * s, m), wg.reshape(1, m, e),
                             w_packed=wg_p).reshape(g, s, e)
  gating = hp.moe_gating
  z = hp.moe_z_loss if gating == "switch" else None
  if gating == "top_2":
    r = hip.top2_gating(logits, c, importance=imp, num_microbatches=mb)
  elif gating == "ntlb":
    r = hip.ntlb_gating(logits, c, hp.moe_ntlb_top_k, importance=imp,
                        num_microbatches=mb)
  else:
    r = hip.switch_gating(logits, c, importance=imp, z_loss=z,
                          num_microbatches=mb,
                          slots_by_gate=gating == "switch_max")
  expert_in = hip.dispatch(xg, r)
  h = torch.empty((e, g * c, hdim), dtype=xg.dtype, device="cuda")
  y = hip.expert_ffn(expert_in.reshape(e, g * c, m), wi_p, wo_p, "relu", h=h)
  # backward
  dout = H.to_gpu(d_out, act_dtype)
  dy, dgate = hip.combine_backward(dout, y.reshape(e, g, c, n), r)
  dxe, dwi, dwo = hip.expert_ffn_backward(
      expert_in.reshape(e, g * c, m), h, dy.reshape(e, g * c, n), wi, wo, "relu")
  dl = torch.tensor([d_loss], dtype=H.ACT_TORCH[act_dtype]).float().cuda()
  scale = torch.tensor(hp.moe_loss_coef, dtype=H.ACT_TORCH[act_dtype]).item()
  dlogits = hip.gating_backward(
      logits, r, dgate, dl, scale,
      router="switch" if gating == "switch_max" else gating,
      top_k=hp.moe_ntlb_top_k, importance=imp, z_loss=z, num_microbatches=mb)
  dwg = hip.router_backward_weights(xg.reshape(g * s, m),
                                    dlogits.reshape(g * s, e))
  dx = hip.dispatch_backward(dxe.reshape(e, g, c, m), r, s, dlogits,
                             wg_p.reshape(e, m))
  return dict(dx=H.to_np(dx), dw_gate=H.to_np(dwg), dwi=H.to_np(dwi),
              dwo=H.to_np(dwo), dlogits=H.to_np(dlogits), dgate=H.to_np(dgate))


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(700, 128, 8), (1030, 256, 64), (96, 384, 72),
                                   (513, 128, 40), (200, 72, 6)])
def test_router_backward_weights(hip, shape, act_dtype):
  """dw_gate = x^T . dlogits against a float64 product: the float32
  matrix-core kernel (M a multiple of 128, E of 8) and the plain one."""
  t, m, e = shape
  rng = np.random.default_rng(t + m + e)
  x = O.cast_act(rng.standard_normal((t, m)).astype(np.float32), act_dtype)
  dl = (rng.standard_normal((t, e)) * 0.1).astype(np.float32)
  got = H.to_np(hip.router_backward_weights(
      H.to_gpu(x, act_dtype), torch.from_numpy(dl).cuda()))
  want = x.astype(np.float64).T @ dl.astype(np.float64)
  tol = H.value_tolerance(act_dtype)
  np.testing.assert_allclose(got, O.cast_act(want.astype(np.float32), act_dtype),
                             rtol=tol["rtol"],
                             atol=tol["atol"] * np.abs(want).max())


CASES = [
    # gating, G, S, M, H, E, cf, dtype, nonpadding
    ("top_2", 2, 64, 16, 24, 4, 1.0, "float32", True),
    ("top_2", 3, 50, 24, 40, 5, 1.25, "float32", False),
    ("top_2", 2, 128, 64, 128, 8, 1.0, "bfloat16", True),
    ("switch", 2, 64, 16, 24, 4, 1.0, "float32", True),
    ("switch", 2, 128, 64, 128, 8, 1.25, "bfloat16", False),
    ("switch_max", 2, 64, 16, 24, 4, 0.75, "float32", True),
    ("top_2", 2, 256, 256, 512, 8, 1.0, "bfloat16", True),   # MFMA GEMM paths
    ("ntlb", 2, 96, 16, 24, 6, 1.0, "float32", True),
    ("ntlb", 2, 128, 64, 128, 8, 0.75, "bfloat16", False),
]


@pytest.mark.parametrize("case", CASES, ids=[
    "%s-%s-%d" % (c[0], c[7], i) for i, c in enumerate(CASES)])
def test_backward_matches_oracle(hip, case):
  gating, g, s, m, hdim, e, cf, act_dtype, use_np = case
  rng = np.random.default_rng(71)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  if gating == "ntlb":
    w["w_gate"][:, 0] *= 3.0          # a popular expert: later passes matter
  x = H.safe_tokens(rng, g * s, m, w["w_gate"], act_dtype,
                    top=4 if gating == "ntlb" else 3).reshape(g, s, m)
  nonpad = (rng.random((g, s)) < 0.85).astype(np.float32) if use_np else None
  d_out = O.cast_act(rng.standard_normal((g, s, m)).astype(np.float32), act_dtype)
  d_loss, mb = 1.5, 2
  hp = _hp(moe_gating=gating, moe_num_experts=e, moe_hidden_size=hdim,
           moe_group_size=s, moe_capacity_factor_train=cf, moe_loss_coef=0.25,
           moe_ntlb_top_k=3,
           moe_z_loss=0.1 if (gating == "switch" and use_np) else None)
  want = O.moe_layer_v1_backward(x, w["w_gate"], w["wi"], w["wo"], hp, True,
                                 act_dtype, d_out, d_loss, nonpadding=nonpad,
                                 num_microbatches=mb)
  if gating == "ntlb":
    assert (want["aux"]["taken_in_pass"] > 0).any()
  got = run_backward(hip, x, w, hp, act_dtype, d_out, d_loss, nonpad, mb)
  tol = H.value_tolerance(act_dtype)
  np.testing.assert_allclose(got["dgate"], want["dgate"], rtol=1e-2 if
                             act_dtype == "bfloat16" else 1e-4, atol=1e-3 if
                             act_dtype == "bfloat16" else 1e-5)
  scale = np.abs(want["dlogits"]).max()
  np.testing.assert_allclose(got["dlogits"], want["dlogits"],
                             rtol=2e-2 if act_dtype == "bfloat16" else 1e-3,
                             atol=(1e-2 if act_dtype == "bfloat16" else 1e-5) * scale)
  for k in ("dx", "dw_gate", "dwi", "dwo"):
    ref = want[k].reshape(got[k].shape)
    atol = tol["atol"] * max(1.0, np.abs(ref).max())
    np.testing.assert_allclose(got[k], ref, rtol=tol["rtol"], atol=atol,
                               err_msg=k)


@pytest.mark.parametrize("use_importance", [False, True])
def test_gating_backward_second_place_loss(hip, use_importance):
  """d(logits) of the balancing loss alone (zero gate gradients), with the
  second-place term: against the oracle, and the term is not negligible."""
  g, s, e, c = 3, 96, 8, 16
  rng = np.random.default_rng(91)
  logits = H.safe_logits(rng, g, s, e, scale=1.5)
  imp = None
  if use_importance:
    imp = rng.choice([0.0, 0.5, 1.0], size=(g, s), p=[0.2, 0.2, 0.6]).astype(np.float32)
  r_o = O.top_2_gating(logits, c, importance=imp, policy="threshold",
                       threshold=0.3, use_second_place_loss=True,
                       num_microbatches=2)
  zeros = np.zeros((g, s), np.float32)
  want = O.gating_backward(logits, r_o, "top_2", zeros, zeros, 0.7, imp, 2,
                           use_second_place_loss=True)
  without = O.gating_backward(logits, r_o, "top_2", zeros, zeros, 0.7, imp, 2)
  assert np.abs(want - without).max() > 0.2 * np.abs(want).max()
  lg = torch.from_numpy(logits).cuda()
  ig = None if imp is None else torch.from_numpy(imp).cuda()
  r = hip.top2_gating(lg, c, importance=ig, policy="threshold", threshold=0.3,
                      use_second_place_loss=True, num_microbatches=2)
  np.testing.assert_allclose(float(r.loss), r_o["loss"], rtol=1e-5)
  dgate = torch.zeros((g, s, 2), dtype=torch.float32, device="cuda")
  dl = torch.tensor([0.7], dtype=torch.float32, device="cuda")
  got = hip.gating_backward(lg, r, dgate, dl, 1.0, router="top_2",
                            importance=ig, num_microbatches=2,
                            use_second_place_loss=True)
  np.testing.assert_allclose(H.to_np(got), want, rtol=1e-3,
                             atol=1e-5 * np.abs(want).max())
  got0 = hip.gating_backward(lg, r, dgate, dl, 1.0, router="top_2",
                             importance=ig, num_microbatches=2)
  np.testing.assert_allclose(H.to_np(got0), without, rtol=1e-3,
                             atol=1e-5 * np.abs(without).max())
