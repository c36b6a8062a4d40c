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


def run_backward(hip, x, w, hp, act_dtype, d_out, d_loss, nonpad, mb,
                 compact=False):
  """The forward and backward call sequence of one v1 layer through the C ABI
  (what MoEV1Operation and its gradient do), on [G, S, M] tokens.  compact: the
  calls that keep every expert's occupied slots at the front of its rows."""
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
                        num_microbatches=mb,
                        softmax_dtype=H.ACT_TORCH[act_dtype])
  else:
    r = hip.switch_gating(logits, c, importance=imp, z_loss=z,
                          num_microbatches=mb,
                          slots_by_gate=gating == "switch_max")
  dout = H.to_gpu(d_out, act_dtype)
  ro = {}
  if compact:
    assert hip.compact_training_applies(xg, r, hdim, n, "relu")
    y, row_offsets, h = hip.compact_expert_ffn(xg, r, wi_p, wo_p, "relu",
                                               want_hidden=True)
    ro = dict(row_offsets=row_offsets)
    expert_in = hip.dispatch(xg, r, **ro)
    dy, dgate = hip.combine_backward(dout, y.reshape(e, g, c, n), r, **ro)
    dxe, dwi, dwo = hip.compact_expert_ffn_backward(
        expert_in.reshape(e, g * c, m), h, dy.reshape(e, g * c, n), wi, wo, r,
        row_offsets, "relu")
  else:
    expert_in = hip.dispatch(xg, r)
    h = torch.empty((e, g * c, hdim), dtype=xg.dtype, device="cuda")
    y = hip.expert_ffn(expert_in.reshape(e, g * c, m), wi_p, wo_p, "relu", h=h)
    dy, dgate = hip.combine_backward(dout, y.reshape(e, g, c, n), r)
    dxe, dwi, dwo = hip.expert_ffn_backward(
        expert_in.reshape(e, g * c, m), h, dy.reshape(e, g * c, n), wi, wo,
        "relu")
  dl = torch.tensor([d_loss], dtype=H.ACT_TORCH[act_dtype]).float().cuda()
  scale = torch.tensor(hp.moe_loss_coef, dtype=H.ACT_TORCH[act_dtype]).item()
  dlogits = hip.gating_backward(
      logits, r, dgate, dl, scale,
      router="switch" if gating == "switch_max" else gating,
      top_k=hp.moe_ntlb_top_k, importance=imp, z_loss=z, num_microbatches=mb,
      softmax_dtype=(H.ACT_TORCH[act_dtype] if gating == "ntlb"
                     else torch.float32))
  dwg = hip.router_backward_weights(xg.reshape(g * s, m),
                                    dlogits.reshape(g * s, e))
  dx = hip.dispatch_backward(dxe.reshape(e, g, c, m), r, s, dlogits,
                             wg_p.reshape(e, m), w_gate=wg.reshape(m, e), **ro)
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
    # the router's share of d(tokens) on the matrix cores (512 columns, 16 experts)
    ("top_2", 2, 256, 512, 256, 16, 1.0, "bfloat16", True),
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
                    top=4 if gating == "ntlb" else 3,
                    bf16_router=(gating == "ntlb" and act_dtype == "bfloat16")
                    ).reshape(g, s, m)
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


def test_router_backward_weights_repeats_bit_for_bit(hip):
  """bfloat16 tokens at widths the bfloat16 matrix-core kernel takes: the sums
  over the token chunks run in a fixed order, so two calls give the same bits
  (and the float64 product to rounding)."""
  t, m, e = 10000, 512, 64
  gen = torch.Generator(device="cuda").manual_seed(3)
  x = torch.randn((t, m), generator=gen, device="cuda").to(torch.bfloat16)
  dl = torch.randn((t, e), generator=gen, device="cuda") * 0.1
  a = hip.router_backward_weights(x, dl)
  b = hip.router_backward_weights(x, dl)
  assert torch.equal(a, b)
  want = x.double().t() @ dl.double()
  err = (a.double() - want).abs()
  assert bool((err <= want.abs() * 2.0 ** -8 * 1.01 + 1e-4).all())


COMPACT_CASES = [
    # gating, G, S, M, H, E, capacity factor, padding mask
    ("switch", 4, 512, 256, 512, 8, 2.0, True),
    ("switch", 2, 1024, 256, 256, 4, 1.25, False),   # 640 rows per expert
    ("ntlb", 4, 512, 256, 512, 8, 2.0, False),
    ("switch_max", 4, 512, 256, 512, 8, 2.0, True),
]


@pytest.mark.parametrize("case", COMPACT_CASES, ids=[
    "%s-%d" % (c[0], i) for i, c in enumerate(COMPACT_CASES)])
def test_compact_backward_matches_oracle(hip, case):
  """The gradient calls on compacted rows (one choice per token: the occupied
  slots at the front of every expert's rows, the GEMMs over those only)
  against the oracle's backward, and against the padded call sequence: the
  token gradient bit for bit (every row's sums run in the same order), the
  expert kernels' gradients to rounding (their sums over token rows are split
  into other K tiles)."""
  gating, g, s, m, hdim, e, cf, use_np = case
  act_dtype = "bfloat16"
  rng = np.random.default_rng(73)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  w["w_gate"][:, 0] *= 2.0          # a popular expert (overflows) ...
  w["w_gate"][:, 1] *= 0.25         # ... and one few tokens choose
  x = H.safe_tokens(rng, g * s, m, w["w_gate"], act_dtype,
                    top=4 if gating == "ntlb" else 3,
                    bf16_router=(gating == "ntlb" and act_dtype == "bfloat16")
                    ).reshape(g, s, m)
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
  got = run_backward(hip, x, w, hp, act_dtype, d_out, d_loss, nonpad, mb,
                     compact=True)
  padded = run_backward(hip, x, w, hp, act_dtype, d_out, d_loss, nonpad, mb)
  for k in ("dx", "dgate", "dlogits"):
    np.testing.assert_array_equal(got[k], padded[k], err_msg=k)
  for k in ("dwi", "dwo", "dw_gate"):   # (the router's sums: atomic adds)
    np.testing.assert_allclose(got[k], padded[k], rtol=2e-2,
                               atol=2e-3 * np.abs(padded[k]).max(), err_msg=k)
  tol = H.value_tolerance(act_dtype)
  for k in ("dx", "dw_gate", "dwi", "dwo"):
    ref = want[k].reshape(got[k].shape)
    atol = tol["atol"] * max(1.0, np.abs(ref).max())
    np.testing.assert_allclose(got[k], ref, rtol=tol["rtol"], atol=atol,
                               err_msg=k)


def test_compact_gradient_calls_edge_fills(hip):
  """Row counts per expert chosen by hand: none (its kernels' gradients are
  exactly zero), one, a whole 256-row tile, every row, and counts that end
  inside a K tile of 64; each compacted call against its padded counterpart
  at the occupied slots, bit for bit where the sums run in the same order."""
  g, s, e, c, m, hdim = 2, 1024, 8, 256, 256, 512
  counts = np.array([[128, 0, 256, 1, 100, 200, 255, 84],
                     [128, 0, 256, 0, 91, 256, 255, 38]])
  assert (counts.sum(1) == s).all() and (counts <= c).all()
  rng = np.random.default_rng(5)
  logits = 0.01 * rng.standard_normal((g, s, e)).astype(np.float32)
  for gi in range(g):
    owner = rng.permutation(np.repeat(np.arange(e), counts[gi]))
    logits[gi, np.arange(s), owner] += 6.0
  lg = torch.from_numpy(logits).cuda()
  r = hip.switch_gating(lg, c)
  fill = H.to_np(r.fill)
  np.testing.assert_array_equal(fill, counts)
  dt = torch.bfloat16
  gen = torch.Generator(device="cuda").manual_seed(9)
  def rand(*shape, scale=1.0):
    return (torch.randn(shape, device="cuda", generator=gen) * scale).to(dt)
  xg = rand(g, s, m)
  wi, wo = rand(e, m, hdim, scale=m ** -0.5), rand(e, hdim, m, scale=hdim ** -0.5)
  wi_p, wo_p = hip.pack_weights(wi, dt), hip.pack_weights(wo, dt)
  dout = rand(g, s, m)
  assert hip.compact_training_applies(xg, r, hdim, m, "relu")
  y_c, ro, h_c = hip.compact_expert_ffn(xg, r, wi_p, wo_p, "relu",
                                        want_hidden=True)
  want_ro = np.concatenate([np.zeros((e, 1), np.int64),
                            np.cumsum(counts.T, axis=1)[:, :-1]], axis=1)
  np.testing.assert_array_equal(H.to_np(ro), want_ro)
  xe_c = hip.dispatch(xg, r, row_offsets=ro).reshape(e, g * c, m)
  xe_p = hip.dispatch(xg, r).reshape(e, g, c, m)
  h_p = torch.empty((e, g * c, hdim), dtype=dt, device="cuda")
  y_p = hip.expert_ffn(xe_p.reshape(e, g * c, m), wi_p, wo_p, "relu", h=h_p)
  dy_c, dgate_c = hip.combine_backward(dout, y_c.reshape(e, g, c, m), r,
                                       row_offsets=ro)
  dy_p, dgate_p = hip.combine_backward(dout, y_p.reshape(e, g, c, m), r)
  dxe_c, dwi_c, dwo_c = hip.compact_expert_ffn_backward(
      xe_c, h_c, dy_c.reshape(e, g * c, m), wi, wo, r, ro, "relu")
  dxe_p, dwi_p, dwo_p = hip.expert_ffn_backward(
      xe_p.reshape(e, g * c, m), h_p, dy_p.reshape(e, g * c, m), wi, wo, "relu")
  dx_c = hip.dispatch_backward(dxe_c.reshape(e, g, c, m), r, s, row_offsets=ro)
  dx_p = hip.dispatch_backward(dxe_p.reshape(e, g, c, m), r, s)

  def occupied(t_c, t_p):
    """(compacted rows, the same slots of the padded tensor) per expert."""
    t_c = t_c.reshape(e, g * c, -1)
    t_p = t_p.reshape(e, g, c, -1)
    for ei in range(e):
      rows = torch.cat([t_p[ei, gi, :counts[gi, ei]] for gi in range(g)])
      yield ei, t_c[ei, :rows.shape[0]], rows
  for name, t_c, t_p in (("expert_in", xe_c, xe_p), ("h", h_c, h_p),
                         ("y", y_c, y_p), ("dy", dy_c, dy_p),
                         ("dexpert_in", dxe_c, dxe_p)):
    for ei, a, b in occupied(t_c, t_p):
      assert torch.equal(a, b), (name, ei)
  # the zero rows up to the end of the last occupied 256-row tile
  for t_c in (xe_c, dy_c.reshape(e, g * c, m)):
    for ei in range(e):
      used = int(counts[:, ei].sum())
      end = min(g * c, -(-used // 256) * 256)
      assert not t_c[ei, used:end].any(), ei
  assert torch.equal(dgate_c, dgate_p)
  assert torch.equal(dx_c, dx_p)
  assert not dwi_c[1].any() and not dwo_c[1].any()    # the expert without rows
  for name, a, b in (("dwi", dwi_c, dwi_p), ("dwo", dwo_c, dwo_p)):
    a, b = a.float(), b.float()
    assert torch.isfinite(a).all(), name
    np.testing.assert_allclose(H.to_np(a), H.to_np(b), rtol=2e-2,
                               atol=2e-3 * float(b.abs().max()), err_msg=name)
  # against float64 sums over the occupied rows
  for ei, xa, _ in occupied(xe_c, xe_p):
    used = xa.shape[0]
    hd = h_c[ei, :used].double()
    dyd = dy_c.reshape(e, g * c, m)[ei, :used].double()
    dh = (dyd @ wo[ei].double().T) * (hd > 0)
    np.testing.assert_allclose(
        H.to_np(dwo_c[ei].float()), H.to_np((hd.T @ dyd).float()), rtol=2e-2,
        atol=1e-2 * max(1e-6, float((hd.T @ dyd).abs().max())), err_msg=str(ei))
    np.testing.assert_allclose(
        H.to_np(dwi_c[ei].float()), H.to_np((xa.double().T @ dh).float()),
        rtol=2e-2, atol=1e-2 * max(1e-6, float((xa.double().T @ dh).abs().max())),
        err_msg=str(ei))


@pytest.mark.parametrize("shape", [(4, 512, 1024, 64, 12), (3, 96, 512, 16, 8),
                                   (2, 64, 1536, 128, 1), (2, 64, 512, 48, 4),
                                   (1, 96, 256, 80, 3), (3, 32, 768, 112, 1)],
                         ids=lambda s: "x".join(map(str, s)))
def test_dispatch_backward_router_share_on_matrix_cores(hip, shape):
  """d(tokens) = the rows of d(expert_in) + d(logits) . w_gate^T with the
  second term on the bfloat16 matrix cores (d(logits) as two bfloat16 terms):
  against float64 arithmetic rounded once, and against the kernel that does
  the term in float32 multiply-adds (equal up to one rounding step of the
  result)."""
  g, s, m, e, c = shape
  dt = torch.bfloat16
  gen = torch.Generator(device="cuda").manual_seed(17)
  mk = lambda *sh: torch.randn(sh, generator=gen, device="cuda")
  r = hip.top2_gating(mk(g, s, e), c)
  dxe = mk(e, g, c, m).to(dt)
  dlogits = mk(g, s, e) * 3.0
  w = (mk(m, e) / m ** 0.5).to(dt)
  w_p = hip.pack_weights(w.reshape(1, m, e), dt).reshape(e, m)
  got = hip.dispatch_backward(dxe, r, s, dlogits, w_p, w_gate=w)
  plain = hip.dispatch_backward(dxe, r, s, dlogits, w_p)
  # float64 reference
  idx, pos = r.idx.long(), r.pos.long()
  on = (r.kept != 0) & (r.gate.to(dt) != 0)
  gi = torch.arange(g, device="cuda").view(g, 1, 1).expand(g, s, 2)
  rows = dxe.double()[idx, gi, pos.clamp(0, c - 1)] * on.unsqueeze(-1)
  want = rows.sum(2) + dlogits.double() @ w.double().t()
  assert on.any() and not on.all()
  err = (got.double() - want).abs()
  # one rounding of the result (half a unit in the last place of bfloat16)
  # on top of float32 sums of terms of size ~10
  assert bool((err <= want.abs() * 2.0 ** -8 * 1.01 + 2e-5).all())
  step = (got.float() - plain.float()).abs()
  assert bool((step <= plain.float().abs() * 2.0 ** -7 + 4e-5).all())
  assert float((step > 0).float().mean()) < 0.02


def test_full_size_router_terms_on_matrix_cores(hip):
  """Configuration 4's token count and widths (65536 tokens, d_model 4096, 64
  experts).  The router kernel's gradient from bfloat16 tokens (d(logits) as
  two bfloat16 terms on the bfloat16 matrix cores) against the same product
  from the tokens widened to float32 (float32 matrix cores); the router's
  share of d(tokens) on the matrix cores against the kernel with float32
  multiply-adds.  Each pair equal up to one rounding step of the bfloat16
  result."""
  g, s, m, e, c = 32, 2048, 4096, 64, 64
  dt = torch.bfloat16
  gen = torch.Generator(device="cuda").manual_seed(41)
  mk = lambda *sh: torch.randn(sh, generator=gen, device="cuda")
  x = mk(g * s, m).to(dt)
  dlogits = mk(g, s, e) * 0.05
  dw = hip.router_backward_weights(x, dlogits.reshape(g * s, e)).float()
  dw32 = hip.router_backward_weights(x.float(), dlogits.reshape(g * s, e))
  scale = float(dw32.abs().max())
  assert float((dw - dw32).abs().max()) <= scale * 2.0 ** -8 * 1.01
  assert float((dw - dw32).abs().mean()) <= float(dw32.abs().mean()) * 2.0 ** -9
  del x, dw, dw32
  route = mk(g, s, e)
  route[..., 0] += 2.0         # an expert that overflows on first choices
  r = hip.top2_gating(route, c)
  dxe = mk(e, g, c, m).to(dt)
  w = (mk(m, e) / m ** 0.5).to(dt)
  w_p = hip.pack_weights(w.reshape(1, m, e), dt).reshape(e, m)
  got = hip.dispatch_backward(dxe, r, s, dlogits, w_p, w_gate=w).float()
  plain = hip.dispatch_backward(dxe, r, s, dlogits, w_p).float()
  step = (got - plain).abs()
  assert bool((step <= plain.abs() * 2.0 ** -7 + 4e-5).all())
  assert float((step > 0).float().mean()) < 0.02
  # a token no expert keeps gets the router's share alone
  lost = ~(r.kept != 0).any(-1)
  assert bool(lost.any())
  share = dlogits[lost].double() @ w.double().t()
  assert float((got[lost].double() - share).abs().max()) <= float(
      share.abs().max()) * 2.0 ** -8 * 1.01


def test_full_size_compact_backward(hip):
  """Eight experts of configuration 4 at their real sizes (32 groups, capacity
  64: 2048 slot rows per expert, d_model 4096, d_ff 16384) behind a switch
  router that fills one expert and a third of the others: the compacted calls
  against the padded ones.  Token gradients and gate gradients bit for bit;
  the experts' kernel gradients to rounding; every occupied row of the
  intermediate tensors bit for bit."""
  g, s, e, c, m, hdim = 32, 256, 8, 64, 4096, 16384
  dt = torch.bfloat16
  gen = torch.Generator(device="cuda").manual_seed(31)
  mk = lambda *shape: torch.randn(shape, generator=gen, device="cuda")
  logits = mk(g, s, e)
  logits[..., 0] += 1.2        # a popular expert: some of its groups overflow
  r = hip.switch_gating(logits, c)
  fill = r.fill.cpu().numpy()
  used = fill.sum(0)
  # (one expert with every slot taken, the others about a third full)
  assert (fill < c).any() and (fill == c).any() and used.min() < g * c // 2
  xg = mk(g, s, m).to(dt)
  wi = (mk(e, m, hdim) / m ** 0.5).to(dt)
  wo = (mk(e, hdim, m) / hdim ** 0.5).to(dt)
  dout = mk(g, s, m).to(dt)
  wi_p, wo_p = hip.pack_weights(wi, dt), hip.pack_weights(wo, dt)
  assert hip.compact_training_applies(xg, r, hdim, m, "relu")
  y_c, ro, h_c = hip.compact_expert_ffn(xg, r, wi_p, wo_p, "relu",
                                        want_hidden=True)
  xe_c = hip.dispatch(xg, r, row_offsets=ro).reshape(e, g * c, m)
  dy_c, dgate_c = hip.combine_backward(dout, y_c.reshape(e, g, c, m), r,
                                       row_offsets=ro)
  dxe_c, dwi_c, dwo_c = hip.compact_expert_ffn_backward(
      xe_c, h_c, dy_c.reshape(e, g * c, m), wi, wo, r, ro, "relu")
  dx_c = hip.dispatch_backward(dxe_c.reshape(e, g, c, m), r, s, row_offsets=ro)
  del y_c, dxe_c
  xe_p = hip.dispatch(xg, r).reshape(e, g * c, m)
  h_p = torch.empty((e, g * c, hdim), dtype=dt, device="cuda")
  y_p = hip.expert_ffn(xe_p, wi_p, wo_p, "relu", h=h_p)
  dy_p, dgate_p = hip.combine_backward(dout, y_p.reshape(e, g, c, m), r)
  dxe_p, dwi_p, dwo_p = hip.expert_ffn_backward(
      xe_p, h_p, dy_p.reshape(e, g * c, m), wi, wo, "relu")
  dx_p = hip.dispatch_backward(dxe_p.reshape(e, g, c, m), r, s)
  assert torch.equal(dx_c, dx_p) and torch.equal(dgate_c, dgate_p)
  assert dx_c.abs().sum() > 0
  # the hidden tensor's occupied rows, expert by expert
  for ei in (0, e - 1):
    rows = torch.cat([h_p.reshape(e, g, c, hdim)[ei, gi, :fill[gi, ei]]
                      for gi in range(g)])
    assert torch.equal(h_c[ei, :rows.shape[0]], rows)
  for name, a, b in (("dwi", dwi_c, dwi_p), ("dwo", dwo_c, dwo_p)):
    a, b = a.float(), b.float()
    assert bool(torch.isfinite(a).all()), name
    err = (a - b).abs().max().item()
    assert err <= 2e-2 * b.abs().max().item(), (name, err)
    assert (a - b).abs().mean().item() <= 2e-3 * b.abs().mean().item(), name


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
