"""End-to-end GPU parity of the layers, called through the mtf-shaped API on
HipMeshImpl, against the CPU oracle on the same seeded inputs."""

import numpy as np
import pytest
import torch

import mesh_amd as mtf
from mesh_amd.transformer import moe
from oracle import moe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


def make_hparams(**kw):
  hp = dict(
      moe_gating="top_2", moe_num_experts=8, moe_loss_coef=1e-2,
      moe_hidden_size=64, moe_group_size=32, moe_min_expert_capacity=4,
      moe_capacity_factor_train=1.25, moe_capacity_factor_eval=2.0,
      moe_capacity_factor_second_level=1.0, moe_use_second_place_loss=False,
      moe_second_policy_train="all", moe_second_policy_eval="all",
      moe_second_threshold_train=0.2, moe_second_threshold_eval=0.2,
      moe_dropout_rate=0.0, moe_use_experts_attention=False)
  hp.update(kw)
  return moe.HParams(**hp), O.HParams(**hp)


def run_v1(x, weights, hp, train, act_dtype, nonpadding=None, activation="relu",
           num_microbatches=None, variable_dtype=None):
  """x: float32 array [batch, length, M] of activation-dtype values."""
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  b, l, m = x.shape
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  npad = None
  if nonpadding is not None:
    npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpadding).to(dt),
                                mtf.Shape(dims[:2]))
  n = weights["wo"].shape[-1]
  vdt = variable_dtype or mtf.VariableDType(torch.float32, torch.float32, dt)
  with mtf.variable_scope("moe"):
    y, loss = moe.transformer_moe_layer_v1(
        xt, mtf.Dimension("d_model", n), hp, train, vdt, nonpadding=npad,
        activation=activation, num_microbatches=num_microbatches)
  router = {"switch": "switch_gating", "switch_max": "switch_max_gating",
            "ntlb": "ntlb_gating",
            "expert_selection": "expert_selection_gating"}.get(
                hp.moe_gating, "top_2_gating")
  init = {"moe/%s/kernel" % router: weights["w_gate"],
          "moe/wo/kernel": weights["wo"]}
  if isinstance(weights["wi"], list):
    init.update(("moe/wi_%d/kernel" % i, v) for i, v in enumerate(weights["wi"]))
  else:
    init["moe/wi/kernel"] = weights["wi"]
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  out = H.to_np(lowering.export_to_tf_tensor(y))
  return out, float(H.to_np(lowering.export_to_tf_tensor(loss))), lowering, (xt, y)


V1_CASES = [
    # name, batch, length, M, H, E, group, cf, dtype
    ("tiny_f32", 2, 64, 16, 64, 8, 32, 1.25, "float32"),
    ("tiny_bf16", 2, 64, 16, 64, 8, 32, 1.25, "bfloat16"),
    ("ragged_f32", 3, 50, 24, 40, 5, 64, 1.0, "float32"),
    ("cfg1_f32", 2, 1024, 512, 2048, 8, 1024, 1.25, "float32"),
    ("cfg2_quarter_bf16", 4, 1024, 1024, 4096, 32, 1024, 1.25, "bfloat16"),
]


@pytest.mark.parametrize("case", V1_CASES, ids=[c[0] for c in V1_CASES])
def test_v1_matches_oracle(case):
  _, b, l, m, hdim, e, group, cf, act_dtype = case
  rng = np.random.default_rng(101)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype).reshape(b, l, m)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_train=cf)
  got, got_loss, _, _ = run_v1(x, w, hp, True, act_dtype)
  want, want_loss, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                        True, act_dtype, dense=b * l <= 4096)
  assert aux["kept_1"].mean() < 1.0 or cf > 1.2   # the drop path is exercised
  np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-2 if act_dtype == "bfloat16" else 1e-5)


def test_v1_closed_form_layer():
  """A layer whose output has a closed form, no oracle involved: expert e
  multiplies by a_e > 0 (wi_e = a_e I, wo_e = I), the router reads the first E
  channels, capacity is ample, so
    out[t] = (g1 a_i1 + g2 a_i2) relu(x[t])
  with (i1, i2) the two largest routing channels of the token and g the top-2
  softmax gates normalised by their sum (moe.py:1397-1415, :509-510), and
    loss = coef E^2 mean_{group, e}(mean_s p . mean_s [i1 = e])   (:1420-1442).
  Evaluated in float64."""
  b, l, m, e, group = 2, 32, 16, 4, 32
  rng = np.random.default_rng(7)
  a = np.array([0.5, 1.0, 1.5, 2.0])
  eye = np.eye(m, dtype=np.float32)
  w_gate = np.zeros((m, e), np.float32)
  w_gate[:e] = 2.0 * np.eye(e)
  w = dict(w_gate=w_gate, wi=np.stack([a_e * eye for a_e in a]).astype(np.float32),
           wo=np.stack([eye] * e))
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  # routing channels: a permutation of well separated levels per token
  levels = np.array([1.5, 0.9, 0.3, -0.3], np.float32)
  for bi in range(b):
    for t in range(l):
      x[bi, t, :e] = rng.permutation(levels)
  hp, _ = make_hparams(moe_num_experts=e, moe_hidden_size=m, moe_group_size=group,
                       moe_capacity_factor_eval=float(e))
  got, got_loss, _, _ = run_v1(x, w, hp, False, "float32")
  logits = 2.0 * x[..., :e].astype(np.float64)
  prob = np.exp(logits - logits.max(-1, keepdims=True))
  prob /= prob.sum(-1, keepdims=True)
  order = np.argsort(-logits, axis=-1)
  i1, i2 = order[..., 0], order[..., 1]
  p1 = np.take_along_axis(prob, i1[..., None], -1)[..., 0]
  p2 = np.take_along_axis(prob, i2[..., None], -1)[..., 0]
  g1, g2 = p1 / (p1 + p2 + 1e-9), p2 / (p1 + p2 + 1e-9)
  want = (g1 * a[i1] + g2 * a[i2])[..., None] * np.maximum(x.astype(np.float64), 0)
  np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-6)
  # groups are the batch rows here (group size = length)
  density = np.stack([(i1 == k).mean(-1) for k in range(e)], -1)     # [b, e]
  want_loss = 1e-2 * e * e * (prob.mean(1) * density).mean()
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-5)


def test_v1_skewed_routing_drops_tokens():
  """Capacity factor 1.0 with a Zipf-biased router (folded into the router
  weights through a constant input column) overflows the popular experts."""
  b, l, m, hdim, e = 4, 512, 64, 128, 16
  rng = np.random.default_rng(103)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  w["w_gate"][0] = H.zipf_bias(rng, e)
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], "bfloat16",
                    ones_column=True).reshape(b, l, m)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=512, moe_capacity_factor_train=1.0)
  got, _, _, _ = run_v1(x, w, hp, True, "bfloat16")
  want, _, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                                "bfloat16", dense=True)
  assert aux["kept_1"].mean() < 0.9 and aux["kept_2"].mean() < 0.8
  dropped = ~(aux["kept_1"] | aux["kept_2"]).reshape(got.shape[:2])
  assert dropped.any() and (got[dropped] == 0).all()
  np.testing.assert_allclose(got, want, **H.value_tolerance("bfloat16"))


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_v1_nonpadding_eval_and_policies(act_dtype):
  b, l, m, hdim, e = 2, 96, 32, 64, 4
  rng = np.random.default_rng(107)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype).reshape(b, l, m)
  nonpadding = (rng.random((b, l)) < 0.8).astype(np.float32)
  for policy, thr in (("all", 0.2), ("none", 0.2), ("threshold", 0.35)):
    hp, ohp = make_hparams(
        moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=48,
        moe_second_policy_eval=policy, moe_second_threshold_eval=thr,
        moe_use_second_place_loss=True, moe_capacity_factor_eval=1.5)
    got, got_loss, _, _ = run_v1(x, w, hp, False, act_dtype,
                                 nonpadding=nonpadding, activation="gelu",
                                 num_microbatches=2)
    want, want_loss, aux = O.moe_layer_v1(
        x, w["w_gate"], w["wi"], w["wo"], ohp, False, act_dtype,
        nonpadding=nonpadding, activation="gelu", num_microbatches=2)
    if policy == "threshold":
      g2 = O.top_2_gating(aux["logits"], 10 ** 6)["gate_2"]
      assert np.abs(g2 - np.float32(thr)).min() > 1e-5
    np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
    assert (got[nonpadding == 0] == 0).all()
    np.testing.assert_allclose(got_loss, want_loss,
                               rtol=1e-2 if act_dtype == "bfloat16" else 1e-5)


def run_v1_attention(x, weights, hp, train, act_dtype, nonpadding, activation):
  """The layer with moe_use_experts_attention: returns [q, k] arrays."""
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  b, l, m = x.shape
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpadding).to(dt),
                              mtf.Shape(dims[:2]))
  with mtf.variable_scope("moe"):
    outs, _ = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, train,
        mtf.VariableDType(torch.float32, torch.float32, dt), nonpadding=npad,
        activation=activation)
  init = {"moe/top_2_gating/kernel": weights["w_gate"],
          "moe/q_wo/kernel": weights["wo"], "moe/k_wo/kernel": weights["k_wo"]}
  init.update(("moe/wi_%d/kernel" % i, v) for i, v in enumerate(weights["wi"]))
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  return [H.to_np(lowering.export_to_tf_tensor(t)) for t in outs]


@pytest.mark.parametrize("case", [
    (["gelu", "linear"], "float32", "top_2"),
    (["gelu", "linear"], "bfloat16", "top_2"),
    (["linear", "sigmoid"], "bfloat16", "switch"),
    (["relu", "swish", "tanh"], "float32", "expert_selection"),
    (["relu", "linear"], "bfloat16", "top_2+experts_attention")],
    ids=lambda c: "%s-%s-%s" % ("*".join(c[0]), c[1], c[2]))
def test_v1_gated_activations_match_oracle(case):
  """A list of activations: the hidden tensor is the product of one dense layer
  per entry (gated units), variables "wi_0", "wi_1", ..."""
  acts, act_dtype, gating = case
  gating, _, attention = gating.partition("+")
  b, l, m, hdim, e, group = 2, 96, 32, 64, 4, 48
  rng = np.random.default_rng(211)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=[H.normal_weights(rng, (e, m, hdim), m) for _ in acts],
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype).reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.9).astype(np.float32)
  kw = dict(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
            moe_capacity_factor_eval=1.0)
  if gating != "top_2":
    kw.update(SWITCH_HP, moe_gating=gating)
  if attention:
    kw.update(moe_use_experts_attention=True)
    w["k_wo"] = H.normal_weights(rng, (e, hdim, m), hdim)
  hp, ohp = make_hparams(**kw)
  if attention:
    got = run_v1_attention(x, w, hp, False, act_dtype, nonpad, acts)
    want, _, _ = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp, False,
                                act_dtype, nonpadding=nonpad, activation=acts,
                                dense=False, k_wo=w["k_wo"])
    for g_, w_ in zip(got, want):
      np.testing.assert_allclose(g_, w_, **H.value_tolerance(act_dtype))
    return
  got, got_loss, _, _ = run_v1(x, w, hp, False, act_dtype, nonpadding=nonpad,
                               activation=acts)
  want, want_loss, aux = O.moe_layer_v1(
      x, w["w_gate"], w["wi"], w["wo"], ohp, False, act_dtype,
      nonpadding=nonpad, activation=acts, dense=False)
  single, _, _ = O.moe_layer_v1(
      x, w["w_gate"], w["wi"][0], w["wo"], ohp, False, act_dtype,
      nonpadding=nonpad, activation=acts[0], dense=False)
  assert np.abs(want - single).max() > 0.05      # the other factors matter
  np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-2 if act_dtype == "bfloat16" else 1e-5)


def test_v1_rerun_with_new_inputs():
  """Lowering.run(feeds) re-executes the layer with the variables in place."""
  b, l, m, hdim, e = 2, 64, 16, 32, 4
  rng = np.random.default_rng(109)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x1 = H.safe_tokens(rng, b * l, m, w["w_gate"], "float32").reshape(b, l, m)
  x2 = H.safe_tokens(rng, b * l, m, w["w_gate"], "float32").reshape(b, l, m)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim)
  _, _, lowering, (xt, y) = run_v1(x1, w, hp, True, "float32")
  lowering.run({xt: torch.from_numpy(x2)})
  got = H.to_np(lowering.export_to_tf_tensor(y))
  want, _, _ = O.moe_layer_v1(x2, w["w_gate"], w["wi"], w["wo"], ohp, True)
  np.testing.assert_allclose(got, want, **H.value_tolerance("float32"))


def run_v2(x, weights, hp, train, act_dtype, nonpadding=None):
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  names = ["outer_batch", "batch", "length", "d_model"][4 - x.ndim:]
  dims = [mtf.Dimension(nm, s) for nm, s in zip(names, x.shape)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  npad = None
  if nonpadding is not None:
    npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpadding).to(dt),
                                mtf.Shape(dims[:-1]))
  n = weights["wo"].shape[-1]
  vdt = mtf.VariableDType(torch.float32, torch.float32, dt)
  with mtf.variable_scope("moe2d"):
    y, loss = moe.transformer_moe_layer_v2(
        xt, mtf.Dimension("d_model", n), hp, train, vdt, nonpadding=npad)
  init = {"moe2d/outer_gating/kernel": weights["w_outer"],
          "moe2d/inner_gating/kernel": weights["w_inner"],
          "moe2d/wi/kernel": weights["wi"], "moe2d/wo/kernel": weights["wo"]}
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  return (H.to_np(lowering.export_to_tf_tensor(y)),
          float(H.to_np(lowering.export_to_tf_tensor(loss))))


def v2_weights(rng, m, hdim, xe, ye):
  return dict(w_outer=H.normal_weights(rng, (m, xe), m),
              w_inner=H.normal_weights(rng, (xe, m, ye), m),
              wi=H.normal_weights(rng, (ye, xe, m, hdim), m),
              wo=H.normal_weights(rng, (ye, xe, hdim, m), hdim))


def safe_tokens_v2(rng, x, w, act_dtype, min_gap=2e-4):
  """Redraws the rows of x [n_tok, m] whose three largest logits are closer
  than min_gap under the outer router (1e-3 there, as H.safe_tokens) or under
  any outer expert's inner router: whichever slots a token lands in, its inner
  routing then does not depend on the summation order of the projection."""
  routers = [(O.cast_act(w["w_outer"], act_dtype), 1e-3)] + [
      (O.cast_act(wi, act_dtype), min_gap) for wi in w["w_inner"]]
  x = x.copy()
  todo = np.ones(x.shape[0], bool)
  for _ in range(100):
    rows = x[todo]
    bad = np.zeros(rows.shape[0], bool)
    for wr, gap in routers:
      top = -np.sort(-O.router_logits(rows, wr), axis=-1)[..., :3]
      bad |= ((top[..., :-1] - top[..., 1:]) < gap).any(axis=-1)
    where = np.flatnonzero(todo)[bad]
    if where.size == 0:
      return x
    x[where] = O.cast_act(
        rng.standard_normal((where.size, x.shape[1])).astype(np.float32),
        act_dtype)
    todo[:] = False
    todo[where] = True
  raise AssertionError("could not separate the inner router logits")


def inner_gap_ok(aux, min_gap=1e-4):
  """True if no inner-level row that is actually routed has a near-tie."""
  logits = aux["logits_inner"]
  imp = aux["importance_inner"].reshape(logits.shape[:2])
  top = -np.sort(-logits, axis=-1)[..., :3]
  gaps = (top[..., :-1] - top[..., 1:]).min(axis=-1)
  return bool((gaps[imp > 0] > min_gap).all())


V2_CASES = [
    ("f32", (2, 64, 16), 32, 4, 4, 32, 1.25, 1.25, "float32"),
    ("bf16", (2, 64, 16), 32, 4, 4, 32, 1.25, 1.0, "bfloat16"),
    ("outer_batch_f32", (1, 4, 96, 24), 48, 3, 5, 64, 2.0, 1.5, "float32"),
    ("mid_bf16", (8, 256, 128), 256, 4, 8, 256, 1.25, 1.25, "bfloat16"),
    # the expert grid, group size and capacity factors of benchmark
    # configuration 5 (8 x 16 experts, groups of 1024, 1.25 at both levels) on
    # half the tokens and a sixteenth of d_model / hidden size: outer capacity
    # 160, 16 * 160 slots per outer expert -> 2 inner groups of 1280, inner
    # capacity 100
    ("x8y16_bf16", (16, 1024, 128), 512, 8, 16, 1024, 1.25, 1.25, "bfloat16"),
]


@pytest.mark.parametrize("case", V2_CASES, ids=[c[0] for c in V2_CASES])
def test_v2_matches_oracle(case):
  _, shape, hdim, xe, ye, group, cf, cf2, act_dtype = case
  m = shape[-1]
  n_tok = int(np.prod(shape[:-1]))
  hp, ohp = make_hparams(moe_num_experts=[xe, ye], moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_train=cf,
                         moe_capacity_factor_second_level=cf2)
  for seed in range(211, 231):   # first seed without an inner-level near-tie
    rng = np.random.default_rng(seed)
    w = v2_weights(rng, m, hdim, xe, ye)
    x = H.safe_tokens(rng, n_tok, m, w["w_outer"], act_dtype).reshape(shape)
    if n_tok > 4096:
      # too many inner rows for a whole seed to be free of near-ties: redraw
      # the tokens that nearly tie under any outer expert's inner router
      x = safe_tokens_v2(rng, x.reshape(n_tok, m), w, act_dtype).reshape(shape)
    want, want_loss, aux = O.moe_layer_v2(
        x, w["w_outer"], w["w_inner"], w["wi"], w["wo"], ohp, True, act_dtype,
        dense=n_tok <= 1024)
    if inner_gap_ok(aux):
      break
  assert inner_gap_ok(aux)
  got, got_loss = run_v2(x, w, hp, True, act_dtype)
  np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-2 if act_dtype == "bfloat16" else 1e-5)


def _device_normal(fan_in, seed):
  """N(0, 1/sqrt(fan_in)) drawn on the device one leading index at a time."""
  def init(sizes, dtype, device):
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = torch.empty(sizes, dtype=dtype, device=device)
    flat = out.reshape(sizes[0], -1) if len(sizes) > 2 else out.reshape(1, -1)
    for i in range(flat.shape[0]):
      row = torch.randn(flat.shape[1], generator=gen, device=device)
      flat[i] = (row / fan_in ** 0.5).to(dtype)
    return out
  return init


def _gather_combine(y4, r, group_size):
  """combine as a gather in torch: y4 [E, G, C, N], one rounding of
  w1 * y[slot1] + w2 * y[slot2] with the activation-dtype gates."""
  g = r.idx.shape[0]
  idx, kept = r.idx.long(), r.kept.bool()
  pos = r.pos.long().clamp(max=r.capacity - 1)
  w = r.gate.to(y4.dtype).float() * kept.float()
  gi = torch.arange(g, device=y4.device).view(g, 1).expand(g, group_size)
  y1 = y4[idx[..., 0], gi, pos[..., 0]].float()
  y2 = y4[idx[..., 1], gi, pos[..., 1]].float()
  return (w[..., 0:1] * y1 + w[..., 1:2] * y2).to(y4.dtype)


def _float64_balancing_loss(logits, is_one=None):
  """mean over [G, E] of mean_s(p * [imp == 1]) * mean_s(mask_1) * E^2
  (transformer/moe.py:1400-1404, :1420-1424) in float64."""
  p = torch.softmax(logits.double(), dim=-1)
  e = logits.shape[-1]
  mask_1 = torch.nn.functional.one_hot(logits.argmax(-1), e).double()
  if is_one is not None:
    p = p * is_one.double().unsqueeze(-1)
    mask_1 = mask_1 * is_one.double().unsqueeze(-1)
  return float((p.mean(1) * mask_1.mean(1)).mean() * e * e)


def test_v2_cfg5_full_size_properties():
  """Benchmark configuration 5 at full size: transformer_moe_layer_v2 on 32 x
  1024 bf16 tokens, 8 x 16 experts, d_model 2048, hidden 8192, capacity factor
  1.25 at both levels (outer capacity 160; 5120 slots per outer expert -> 5
  inner groups of 1024, inner capacity 80).  The oracle is too slow here, so
  the layer's output is tied, bit for bit, to the library's stages run by hand
  with the logits kept, and each stage is checked through properties: the
  routing records of both levels (slots unique and contiguous, first choices
  before second ones, positions in token order), the inner importance in
  {0, 0.5, 1} with as many of each as the outer level kept first / second
  choices, dispatch and combine against torch gathers, sampled row blocks of
  the experts against float32 matmuls, zero rows for tokens dropped
  everywhere, and both balancing losses against float64."""
  from mesh_amd import moe_hip as hip
  b, l, m, hdim, xe, ye = 32, 1024, 2048, 8192, 8, 16
  s_, c_, h0, t_, d_ = 1024, 160, 5, 1024, 80
  dt = torch.bfloat16
  hp, _ = make_hparams(moe_num_experts=[xe, ye], moe_hidden_size=hdim,
                       moe_group_size=1024, moe_capacity_factor_train=1.25,
                       moe_capacity_factor_second_level=1.25)
  gen = torch.Generator(device="cuda")
  gen.manual_seed(55)
  x_val = torch.randn((b, l, m), generator=gen, device="cuda").to(dt)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, x_val, mtf.Shape(dims))
  with mtf.variable_scope("moe2d"):
    y, loss = moe.transformer_moe_layer_v2(
        xt, dims[-1], hp, True, mtf.VariableDType(dt, dt, dt))
  init = {"moe2d/outer_gating/kernel": _device_normal(m, 2),
          "moe2d/inner_gating/kernel": _device_normal(m, 5),
          "moe2d/wi/kernel": _device_normal(m, 3),
          "moe2d/wo/kernel": _device_normal(hdim, 4)}
  with hip.StageTimer() as timer:
    lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()},
                            initial_values=init)
  out = lowering.export_to_tf_tensor(y)
  got_loss = float(lowering.export_to_tf_tensor(loss).float())
  assert tuple(out.shape) == (b, l, m) and out.dtype == dt
  assert bool(torch.isfinite(out.float()).all())
  rx, ry = timer.routing
  assert (rx.capacity, rx.num_experts, tuple(rx.idx.shape)) == (c_, xe, (b, s_, 2))
  assert (ry.capacity, ry.num_experts, tuple(ry.idx.shape)) == (
      d_, ye, (xe * h0, t_, 2))
  var = {v.name: lv for v, lv in lowering.variables.items()}
  w_outer = var["moe2d/outer_gating/kernel"].master            # [m, x]
  w_inner = var["moe2d/inner_gating/kernel"].master            # [x, m, y]
  wi_p = var["moe2d/wi/kernel"].packed(dt)                     # [y*x, hidden, m]
  wo_p = var["moe2d/wo/kernel"].packed(dt)                     # [y*x, m, hidden]

  def same_record(a, b_):
    return all(torch.equal(getattr(a, k), getattr(b_, k))
               for k in ("idx", "pos", "gate", "kept", "fill", "loss"))

  # ---- outer level
  xg = x_val.reshape(b, s_, m)
  rx2, logits_x = hip.router_top2_gating(
      xg.reshape(1, b * s_, m), hip.pack_weights(w_outer.reshape(1, m, xe), dt),
      s_, c_, want_logits=True)
  assert same_record(rx, rx2)
  torch.testing.assert_close(logits_x.reshape(b * s_, xe),
                             xg.reshape(-1, m).float() @ w_outer.float(),
                             rtol=1e-4, atol=1e-4)
  used_x = H.assert_routing_properties(rx, logits_x)
  assert not bool(rx.kept.bool().all())                 # some outer drops
  kept_x = rx.kept.bool()
  w_x = rx.gate.to(dt).float() * kept_x.float()
  ein_x, slot_gate = hip.dispatch(xg, rx, want_slot_gate=True)
  sel = kept_x & (w_x != 0)
  gi, si, ki = sel.nonzero(as_tuple=True)
  ref = torch.zeros_like(ein_x)
  ref[rx.idx.long()[gi, si, ki], gi, rx.pos.long()[gi, si, ki]] = xg[gi, si]
  assert torch.equal(ein_x, ref)
  ref_gate = torch.zeros_like(slot_gate)
  ref_gate[rx.idx.long()[gi, si, ki], gi, rx.pos.long()[gi, si, ki]] = w_x[gi, si, ki]
  assert torch.equal(slot_gate, ref_gate)
  del ref, ref_gate

  # ---- inner level: importance from the slot weights (moe.py:724-727)
  imp = 0.5 * ((slot_gate > 0.5).float() + (slot_gate > 0).float())
  imp = imp.reshape(xe * h0, t_)
  n_one = int((imp == 1.0).sum())
  n_half = int((imp == 0.5).sum())
  assert n_one + n_half + int((imp == 0).sum()) == imp.numel()
  w1, w2 = w_x[..., 0], w_x[..., 1]
  assert n_one == int((w1 > 0.5).sum())
  assert n_half == int(((w1 > 0) & (w1 <= 0.5)).sum()) + int((w2 > 0).sum())
  assert int((imp == 0).sum()) == int((~used_x).sum()) + int(
      (kept_x & (w_x == 0)).sum())
  inputs_y = ein_x.reshape(xe, h0 * t_, m)
  ry2, logits_y = hip.router_top2_gating(
      inputs_y, hip.pack_weights(w_inner, dt), t_, d_,
      importance=slot_gate.reshape(xe * h0, t_), importance_from_slot_gate=True,
      want_logits=True)
  assert same_record(ry, ry2)
  ref_logits = torch.bmm(inputs_y.float(), w_inner.float())
  torch.testing.assert_close(logits_y.reshape(xe, h0 * t_, ye), ref_logits,
                             rtol=1e-4, atol=1e-4)
  H.assert_routing_properties(ry, logits_y, importance=imp)
  assert not bool(ry.kept.bool()[imp == 1.0].all())     # some inner drops
  ein_y = hip.dispatch(inputs_y.reshape(xe * h0, t_, m), ry)
  kept_y = ry.kept.bool()
  w_y = ry.gate.to(dt).float() * kept_y.float()
  gi, si, ki = (kept_y & (w_y != 0)).nonzero(as_tuple=True)
  ref = torch.zeros_like(ein_y)
  ref[ry.idx.long()[gi, si, ki], gi, ry.pos.long()[gi, si, ki]] = (
      inputs_y.reshape(xe * h0, t_, m)[gi, si])
  assert torch.equal(ein_y, ref)
  del ref

  # ---- experts: rows of (y, x) are that pair's h0 * d slots
  rows = h0 * d_
  ein = ein_y.reshape(ye * xe, rows, m)
  yy = hip.expert_ffn(ein, wi_p, wo_p, "relu")
  for ei, r0 in ((0, 0), (ye * xe // 2, rows // 2 - 37), (ye * xe - 1, rows - 64),
                 (37, 100)):
    xs = ein[ei, r0:r0 + 64].float()
    h_ref = torch.relu(xs @ wi_p[ei].float().t()).to(dt).float()
    y_ref = h_ref @ wo_p[ei].float().t()
    err = (yy[ei, r0:r0 + 64].float() - y_ref).abs().max().item()
    assert err <= 2e-2 * y_ref.abs().max().item(), (ei, r0, err)
  empty = ~(ein != 0).any(-1)
  assert bool(empty.any()) and not bool(yy[empty].any())

  # ---- the two combines, and the layer's output
  out_y = hip.combine(yy.reshape(ye, xe * h0, d_, m), ry, t_)
  assert torch.equal(out_y, _gather_combine(yy.reshape(ye, xe * h0, d_, m), ry, t_))
  out_x = hip.combine(out_y.reshape(xe, b, c_, m), rx, s_)
  assert torch.equal(out_x, _gather_combine(out_y.reshape(xe, b, c_, m), rx, s_))
  assert torch.equal(out_x.reshape(b, l, m), out)
  dropped = ~kept_x.any(-1)
  assert bool(dropped.any()) and not bool(out.reshape(b, s_, m)[dropped].any())
  # a token kept only in slots that the inner level dropped twice is zero too
  slot_live = kept_y.any(-1).reshape(xe, b, c_)             # per outer slot
  pos_x = rx.pos.long().clamp(max=c_ - 1)
  gi = torch.arange(b, device="cuda").view(b, 1, 1).expand(b, s_, 2)
  live = (kept_x & slot_live[rx.idx.long(), gi, pos_x]).any(-1)
  assert bool((~live & ~dropped).any())
  assert not bool(out.reshape(b, s_, m)[~live].any())

  # ---- losses (moe.py:801: (outer + inner) * moe_loss_coef)
  want_x = _float64_balancing_loss(logits_x)
  want_y = _float64_balancing_loss(logits_y, imp == 1.0)
  np.testing.assert_allclose(float(rx.loss), want_x, rtol=1e-4)
  np.testing.assert_allclose(float(ry.loss), want_y, rtol=1e-4)
  np.testing.assert_allclose(got_loss, (want_x + want_y) * 1e-2, rtol=2e-2)


def test_v2_nonpadding():
  shape, hdim, xe, ye = (2, 80, 16), 32, 2, 4
  rng = np.random.default_rng(223)
  w = v2_weights(rng, 16, hdim, xe, ye)
  x = H.safe_tokens(rng, 160, 16, w["w_outer"], "float32").reshape(shape)
  nonpadding = (rng.random(shape[:-1]) < 0.7).astype(np.float32)
  hp, ohp = make_hparams(moe_num_experts=[xe, ye], moe_hidden_size=hdim,
                         moe_group_size=40, moe_capacity_factor_train=2.0,
                         moe_capacity_factor_second_level=2.0)
  want, want_loss, aux = O.moe_layer_v2(
      x, w["w_outer"], w["w_inner"], w["wi"], w["wo"], ohp, True, "float32",
      nonpadding=nonpadding)
  assert inner_gap_ok(aux)
  got, got_loss = run_v2(x, w, hp, True, "float32", nonpadding=nonpadding)
  np.testing.assert_allclose(got, want, **H.value_tolerance("float32"))
  assert (got[nonpadding == 0] == 0).all()
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-5)


# ---- switch gating ------------------------------------------------------------
SWITCH_HP = dict(moe_gating="switch", moe_switch_policy_train="argmax",
                 moe_switch_policy_eval="input_jitter", moe_switch_dropout=0.1,
                 moe_switch_temperature=1.0, moe_switch_jitter=1e-2,
                 moe_z_loss=None)


@pytest.mark.parametrize("case", V1_CASES[:3] + V1_CASES[4:],
                         ids=[c[0] for c in V1_CASES[:3] + V1_CASES[4:]])
def test_v1_switch_matches_oracle(case):
  _, b, l, m, hdim, e, group, cf, act_dtype = case
  rng = np.random.default_rng(301)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype).reshape(b, l, m)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_eval=cf,
                         **SWITCH_HP)
  got, got_loss, _, _ = run_v1(x, w, hp, False, act_dtype)
  want, want_loss, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                        False, act_dtype, dense=b * l <= 4096)
  assert not aux["kept_1"].all()                 # the drop path is exercised
  np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-2 if act_dtype == "bfloat16" else 1e-4)
  # dropped tokens output exactly zero
  assert (got.reshape(-1, m)[~aux["kept_1"].reshape(-1)] == 0).all()


def test_v1_switch_train_z_loss_and_nonpadding():
  b, l, m, hdim, e = 2, 96, 32, 48, 4
  rng = np.random.default_rng(302)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], "float32").reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  kw = dict(SWITCH_HP, moe_z_loss=1e-2)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=64, moe_capacity_factor_train=1.0, **kw)
  got, got_loss, _, _ = run_v1(x, w, hp, True, "float32", nonpadding=nonpad,
                               num_microbatches=2)
  want, want_loss, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                        True, "float32", nonpadding=nonpad,
                                        num_microbatches=2)
  np.testing.assert_allclose(got, want, **H.value_tolerance("float32"))
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-4)
  assert (got[nonpad == 0] == 0).all()
  # the z-loss is part of the loss: without it the value differs
  hp0, _ = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                        moe_group_size=64, moe_capacity_factor_train=1.0,
                        **SWITCH_HP)
  _, loss0, _, _ = run_v1(x, w, hp0, True, "float32", nonpadding=nonpad,
                          num_microbatches=2)
  assert got_loss > loss0


@pytest.mark.parametrize("gating", ["switch", "switch_max", "ntlb",
                                    "expert_selection"])
def test_v1_router_summaries_on_the_lowering(gating):
  """While training the f1 routers log scalars with mtf.scalar_summary
  (moe.py:865-880, :1010-1046, :1149-1165, :1213-1289): they arrive on the
  Lowering under the reference's names with the oracle's values; an evaluation
  graph and the top-2 router log nothing."""
  b, l, m, hdim, e = 2, 128, 32, 48, 4
  rng = np.random.default_rng(311)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], "float32").reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  kw = dict(SWITCH_HP, moe_gating=gating, moe_ntlb_top_k=2,
            moe_z_loss=1e-2 if gating == "switch" else None)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=64, moe_capacity_factor_train=1.0, **kw)
  _, _, low, _ = run_v1(x, w, hp, True, "float32", nonpadding=nonpad,
                        num_microbatches=2)
  _, _, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                             "float32", nonpadding=nonpad, num_microbatches=2)
  groups = b * l // 64
  want = O.router_summaries(aux["logits"], gating, aux,
                            importance=nonpad.reshape(groups, 64), top_k=2,
                            num_microbatches=2)
  got = {k: float(v) for k, v in low.scalar_summaries.items()}
  name = gating + "_gating"
  np.testing.assert_allclose(got[name + "/entropy"], want["entropy"], rtol=1e-4)
  if gating == "expert_selection":
    per = [got["group_token/moe/split/%d" % i] for i in range(64)]
    np.testing.assert_array_equal(per, want["group_token"])
    expected = {name + "/entropy", "aux_loss"}
  else:
    per = [got["experts/moe/split/%d" % i] for i in range(e)]
    np.testing.assert_allclose(per, want["experts"], rtol=1e-6)
    expected = {name + "/entropy", "aux_loss"}
  if gating in ("switch", "switch_max"):
    np.testing.assert_allclose(got["fraction_routed"], want["fraction_routed"],
                               rtol=1e-6)
    np.testing.assert_allclose(got["expert_gate"], want["expert_gate"], rtol=1e-4)
    expected |= {"fraction_routed", "expert_gate"}
  if gating == "switch":
    np.testing.assert_allclose(got[name + "/z_loss"], want["z_loss"], rtol=1e-4)
    # aux_loss is the balancing loss before the z-loss is added (moe.py:1257)
    _, ohp0 = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                           moe_group_size=64, moe_capacity_factor_train=1.0,
                           **dict(kw, moe_z_loss=None))
    _, loss0, _ = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp0, True,
                                 "float32", nonpadding=nonpad, num_microbatches=2)
    np.testing.assert_allclose(got["aux_loss"] * ohp.moe_loss_coef, loss0,
                               rtol=1e-4)
    expected |= {name + "/z_loss"}
  assert {k for k in got if "/split/" not in k} == expected
  # evaluation: nothing is logged; a second run replaces the first run's values
  _, _, low_eval, _ = run_v1(x, w, hp, False, "float32", nonpadding=nonpad)
  assert low_eval.scalar_summaries == {}
  low.run()
  again = {k: float(v) for k, v in low.scalar_summaries.items()}
  assert again == got
  hp2, _ = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                        moe_group_size=64)
  _, _, low2, _ = run_v1(x, w, hp2, True, "float32", nonpadding=nonpad)
  assert low2.scalar_summaries == {}


def test_scalar_summary_operation():
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  a = mtf.import_tf_tensor(mesh, torch.tensor(1.5), mtf.Shape([]))
  b_ = mtf.scalar_summary("loss", a)
  c_ = mtf.scalar_summary("loss", b_ * 2.0)
  low = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()})
  assert float(low.export_to_tf_tensor(c_)) == 3.0
  assert {k: float(v) for k, v in low.scalar_summaries.items()} == {
      "loss": 1.5, "loss_1": 3.0}
  with pytest.raises(ValueError):
    mtf.scalar_summary("v", mtf.import_tf_tensor(
        mesh, torch.zeros(2), mtf.Shape([mtf.Dimension("d", 2)])))


def test_v1_switch_rejections():
  x = np.zeros((1, 32, 16), np.float32)
  w = dict(w_gate=np.zeros((16, 4), np.float32),
           wi=np.zeros((4, 16, 8), np.float32),
           wo=np.zeros((4, 8, 16), np.float32))
  base = dict(moe_num_experts=4, moe_hidden_size=8, moe_group_size=32)
  hp, _ = make_hparams(**dict(base, **dict(SWITCH_HP,
                                          moe_switch_policy_eval="bogus")))
  with pytest.raises(ValueError, match="Unknown Switch gating policy"):
    run_v1(x, w, hp, False, "float32")
  hp, _ = make_hparams(**dict(base, **dict(SWITCH_HP, moe_z_loss=1e-3)))
  with pytest.raises(ValueError, match="moe_z_loss needs"):
    run_v1(x, w, hp, True, "float32")


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_v1_ntlb_matches_oracle(act_dtype):
  """ntlb end to end with a skewed router, so that pass 0 overflows and the
  later passes place tokens; nonpadding masks some tokens out."""
  b, l, m, hdim, e, group, k = 2, 256, 64, 128, 8, 128, 3
  rng = np.random.default_rng(305)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  w["w_gate"][:, 0] *= 3.0                          # expert 0 is popular
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype, top=k + 1,
                    bf16_router=act_dtype == "bfloat16").reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.85).astype(np.float32)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_eval=1.0,
                         moe_ntlb_top_k=k,
                         **dict(SWITCH_HP, moe_gating="ntlb"))
  got, got_loss, _, _ = run_v1(x, w, hp, False, act_dtype, nonpadding=nonpad,
                               num_microbatches=2)
  want, want_loss, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                        False, act_dtype, nonpadding=nonpad,
                                        num_microbatches=2, dense=True)
  assert (aux["taken_in_pass"] > 0).any() and not aux["kept_1"].all()
  np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-2 if act_dtype == "bfloat16" else 1e-4)
  assert (got.reshape(-1, m)[~aux["kept_1"].reshape(-1)] == 0).all()


@pytest.mark.parametrize("case", [
    ("switch", "input_jitter", "float32"), ("switch", "input_jitter", "bfloat16"),
    ("switch", "input_dropout", "float32"), ("ntlb", "input_jitter", "bfloat16"),
    ("switch_max", "input_dropout", "bfloat16"),
    ("switch", "sample", "float32"), ("switch_max", "sample", "bfloat16")],
    ids=lambda c: "-".join(c))
def test_v1_router_input_noise_matches_oracle(case):
  """Training with the perturbing switch policies: the layer draws u ~ U[0,1)
  of the tokens' shape from torch's generator on the device as its first random
  call; re-seeding reproduces the tensor for the oracle."""
  gating, policy, act_dtype = case
  b, l, m, hdim, e, group = 2, 96, 32, 48, 4, 48
  rng = np.random.default_rng(331)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  kw = dict(SWITCH_HP, moe_gating=gating, moe_switch_policy_train=policy,
            moe_switch_jitter=0.25, moe_switch_dropout=0.3, moe_ntlb_top_k=2,
            moe_switch_temperature=1.5)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_train=1.0,
                         **kw)
  torch.manual_seed(99)
  noise = su = None
  if policy == "sample":
    su = torch.rand((b * l // group, group, e), dtype=torch.float32,
                    device="cuda").cpu().numpy()
  else:
    noise = torch.rand((1, b * l, m), dtype=torch.float32,
                       device="cuda").cpu().numpy().reshape(b, l, m)
  x = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
  for _ in range(100):
    want, want_loss, aux = O.moe_layer_v1(
        x, w["w_gate"], w["wi"], w["wo"], ohp, True, act_dtype,
        num_microbatches=2, dense=False, gate_noise=noise, sample_uniform=su)
    if not (gating == "ntlb" and act_dtype == "bfloat16"):
      break
    # the ntlb router rounds its (perturbed) logits to bfloat16 and runs its
    # softmax there: redraw the tokens with a logit at a rounding midpoint,
    # where two summation orders of the projection could part
    lg = aux["logits"].reshape(b * l, e)
    bad = (H.near_bf16_midpoint(lg, 0.02).any(-1)
           | H.bf16_softmax_fragile_rows(lg))
    if not bad.any():
      break
    x.reshape(b * l, m)[bad] = O.cast_act(
        rng.standard_normal((int(bad.sum()), m)).astype(np.float32), act_dtype)
  else:
    raise AssertionError("no tokens away from the rounding midpoints")
  torch.manual_seed(99)
  got, got_loss, _, _ = run_v1(x, w, hp, True, act_dtype, num_microbatches=2)
  assert (aux["gate_mult"] is not None) == (policy != "sample")
  plain, _, aux0 = O.moe_layer_v1(
      x, w["w_gate"], w["wi"], w["wo"],
      make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                   moe_group_size=group, moe_capacity_factor_train=1.0,
                   **dict(kw, moe_switch_policy_train="argmax"))[1],
      True, act_dtype, num_microbatches=2, dense=False)
  assert (aux["index_1"] != aux0["index_1"]).any()    # the noise changed routes
  np.testing.assert_allclose(got, want, **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-2 if act_dtype == "bfloat16" else 1e-4)
  if policy == "sample":
    return          # the eval policy of SWITCH_HP is another one
  # evaluation draws nothing: same result whatever the generator's state
  a, _, _, _ = run_v1(x, w, hp, False, act_dtype)
  torch.manual_seed(5)
  c, _, _, _ = run_v1(x, w, hp, False, act_dtype)
  np.testing.assert_array_equal(a, c)


def test_v1_switch_max_matches_oracle():
  """switch_max end to end.  Which tokens an over-subscribed expert keeps
  depends on gates that the two implementations compute with different exp
  routines: the seed is chosen so that no expert's C-th and (C+1)-th gate are
  within 1e-5 of each other (checked on the oracle's values)."""
  b, l, m, hdim, e, group = 2, 128, 32, 64, 4, 64
  for seed in range(303, 323):
    rng = np.random.default_rng(seed)
    w = dict(w_gate=H.normal_weights(rng, (m, e), m),
             wi=H.normal_weights(rng, (e, m, hdim), m),
             wo=H.normal_weights(rng, (e, hdim, m), hdim))
    x = H.safe_tokens(rng, b * l, m, w["w_gate"], "float32").reshape(b, l, m)
    hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                           moe_group_size=group, moe_capacity_factor_eval=0.75,
                           **dict(SWITCH_HP, moe_gating="switch_max"))
    want, want_loss, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                          False, "float32")
    p = O.softmax(aux["logits"]).max(-1)
    gaps_ok = True
    for gi in range(aux["num_groups"]):
      for ex in range(e):
        v = -np.sort(-p[gi][aux["index_1"][gi] == ex])
        c = aux["capacity"]
        if len(v) > c and (v[c - 1] - v[c]) < 1e-5:
          gaps_ok = False
    if gaps_ok:
      break
  assert gaps_ok and not aux["kept_1"].all()
  got, got_loss, _, _ = run_v1(x, w, hp, False, "float32")
  np.testing.assert_allclose(got, want, **H.value_tolerance("float32"))
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-4)


def test_v1_switch_hidden_dropout_on_compacted_rows():
  """Training forward of a switch layer with moe_dropout_rate at a shape the
  compacted expert rows take: the dropout runs between the two expert products
  on the compacted hidden tensor.  Against the oracle, with the layer's noise
  (its only random call, reproduced) moved from the compacted rows to the
  [E, G, C] slot order the oracle works in."""
  from mesh_amd import moe_hip
  b, l, m, hdim, e, group = 2, 1024, 256, 512, 4, 1024
  rng = np.random.default_rng(121)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], "bfloat16").reshape(b, l, m)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_train=1.0,
                         moe_dropout_rate=0.25, **SWITCH_HP)
  torch.manual_seed(9)
  with moe_hip.StageTimer() as timer:
    got, got_loss, _, _ = run_v1(x, w, hp, True, "bfloat16")
  assert timer.compacted == 1
  torch.manual_seed(9)
  n_groups = b * l // group
  cap = O.expert_capacity(group, 1.0, e, 4)
  hu = torch.rand((e, n_groups * cap, hdim), dtype=torch.bfloat16,
                  device="cuda").float().cpu().numpy()
  _, _, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                             "bfloat16", dense=False, hidden_uniform=hu)
  idx1 = aux["index_1"].reshape(n_groups, group)
  kept1 = aux["kept_1"].reshape(n_groups, group).astype(bool)
  assert not kept1.all()
  padded = np.zeros_like(hu)
  for ex in range(e):
    row = 0
    for gi in range(n_groups):
      n = int((kept1[gi] & (idx1[gi] == ex)).sum())
      padded[ex, gi * cap:gi * cap + n] = hu[ex, row:row + n]
      row += n
  want, want_loss, _ = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                      True, "bfloat16", dense=False,
                                      hidden_uniform=padded)
  plain, _, _ = O.moe_layer_v1(
      x, w["w_gate"], w["wi"], w["wo"],
      make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                   moe_group_size=group, moe_capacity_factor_train=1.0,
                   **SWITCH_HP)[1], True, "bfloat16", dense=False)
  assert np.abs(want - plain).max() > 0.05            # units were dropped
  np.testing.assert_allclose(got, want, **H.value_tolerance("bfloat16"))
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-2)


# ---- gradients through the mtf-shaped API -------------------------------------
@pytest.mark.parametrize("case", [
    ("top_2", "float32", 101), ("top_2", "bfloat16", 102),
    ("switch", "float32", 103), ("switch_max", "float32", 104),
    ("ntlb", "float32", 105), ("switch+input_jitter", "float32", 106),
    ("switch+input_dropout", "bfloat16", 107),
    ("ntlb+input_jitter", "float32", 108),
    ("top_2+hidden_dropout", "float32", 109),
    ("top_2+hidden_dropout", "bfloat16", 110),
    ("switch+hidden_dropout", "float32", 111),
    ("top_2+second_place_loss", "float32", 112),
    ("top_2+second_place_loss", "bfloat16", 113),
    # shapes the matrix-core kernels take: one choice per token keeps the
    # gradient graph on compacted rows
    ("switch+compact", "bfloat16", 114), ("ntlb+compact", "bfloat16", 115),
    ("switch+compact+input_jitter", "bfloat16", 116),
    ("switch+compact+hidden_dropout", "bfloat16", 117),
    # the same sizes behind a top-2 router (padded rows): the dropout's noise
    # rides on the ReLU mask of the dh GEMM
    ("top_2+large+hidden_dropout", "bfloat16", 118),
    # two choices per token on compacted rows too (an expert's slot rows are
    # whole 256-row tiles at these sizes)
    ("top_2+compact", "bfloat16", 119)],
    ids=lambda c: "%s-%s" % (c[0], c[1]))
def test_v1_gradients_match_oracle(case, monkeypatch):
  """mtf.gradients over the layer (outputs and loss) against the oracle's
  backward, which central differences pin in tests/test_oracle.py."""
  gating, act_dtype, seed = case
  gating, _, noise_policy = gating.partition("+")
  compact = noise_policy.startswith("compact")
  large = compact or noise_policy.startswith("large")
  if large:
    noise_policy = noise_policy.partition("+")[2]
  hidden_dropout = noise_policy == "hidden_dropout"
  loss2 = noise_policy == "second_place_loss"
  if hidden_dropout or loss2:
    noise_policy = ""
  b, l, m, hdim, e, group = 2, 64, 32, 48, 4, 32
  compact_calls = []
  if large:
    b, l, m, hdim, e, group = 2, 1024, 256, 512, 4, 1024
  if compact:
    from mesh_amd import moe_hip
    inner = moe_hip.compact_expert_ffn_backward
    def counted(*args, **kwargs):
      compact_calls.append(1)
      return inner(*args, **kwargs)
    monkeypatch.setattr(moe_hip, "compact_expert_ffn_backward", counted)
  rng = np.random.default_rng(seed)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype, top=4,
                    bf16_router=(gating == "ntlb" and act_dtype == "bfloat16")
                    ).reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.85).astype(np.float32)
  d_out = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
  kw = dict(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
            moe_capacity_factor_train=1.0, moe_loss_coef=0.25)
  if gating != "top_2":
    kw.update(SWITCH_HP, moe_gating=gating, moe_ntlb_top_k=3,
              moe_z_loss=0.1 if gating == "switch" else None)
  if noise_policy:
    kw.update(moe_switch_policy_train=noise_policy, moe_switch_jitter=0.25,
              moe_switch_dropout=0.3)
  if hidden_dropout:
    kw.update(moe_dropout_rate=0.25)
  if loss2:
    kw.update(moe_use_second_place_loss=True, moe_second_policy_train="threshold",
              moe_second_threshold_train=0.3)
  hp, ohp = make_hparams(**kw)
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpad).to(dt),
                              mtf.Shape(dims[:2]))
  with mtf.variable_scope("moe"):
    y, loss = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, True, mtf.VariableDType(torch.float32, torch.float32, dt),
        nonpadding=npad, num_microbatches=2)
  variables = graph.trainable_variables
  assert [v.name.split("/")[-2] for v in variables][1:] == ["wi", "wo"]
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(d_out).to(dt), mtf.Shape(dims))
  dlt = mtf.import_tf_tensor(mesh, torch.tensor(1.5, dtype=dt), mtf.Shape([]))
  grads = mtf.gradients([y, loss], [xt] + [v.outputs[0] for v in variables],
                        grad_ys=[dyt, dlt])
  router = {"switch": "switch_gating", "switch_max": "switch_max_gating",
            "ntlb": "ntlb_gating"}.get(gating, "top_2_gating")
  init = {"moe/%s/kernel" % router: w["w_gate"], "moe/wi/kernel": w["wi"],
          "moe/wo/kernel": w["wo"]}
  torch.manual_seed(seed)
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = [H.to_np(lowering.export_to_tf_tensor(g)) for g in grads]
  noise = None
  if noise_policy:         # the layer's first random call, reproduced
    torch.manual_seed(seed)
    noise = torch.rand((1, b * l, m), dtype=torch.float32,
                       device="cuda").cpu().numpy().reshape(b, l, m)
  hu = None
  if hidden_dropout:       # likewise: uniforms of the hidden tensor's shape
    torch.manual_seed(seed)
    cap = O.expert_capacity(group, 1.0, e, 4)
    hu = torch.rand((e, (b * l // group) * cap, hdim), dtype=dt,
                    device="cuda").float().cpu().numpy()
    if compact:
      # the layer drew the noise for the compacted rows (an expert's occupied
      # slots, groups in order, at the front of its rows): move every slot's
      # noise to the slot's place in the [E, G, C] order the oracle uses
      _, _, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                                 act_dtype, nonpadding=nonpad,
                                 num_microbatches=2, dense=False,
                                 hidden_uniform=hu)   # (the routing ignores it)
      n_groups = b * l // group
      fill = np.asarray(aux["fill"]).reshape(n_groups, e)
      padded = np.zeros_like(hu)
      for ex in range(e):
        row = 0
        for gi in range(n_groups):
          n = int(fill[gi, ex])
          padded[ex, gi * cap:gi * cap + n] = hu[ex, row:row + n]
          row += n
      hu = padded
  want = O.moe_layer_v1_backward(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                                 act_dtype, d_out, 1.5, nonpadding=nonpad,
                                 num_microbatches=2, gate_noise=noise,
                                 hidden_uniform=hu)
  assert not (want["aux"]["kept_1"] | want["aux"]["kept_2"]).all()
  if hidden_dropout:
    out_got = H.to_np(lowering.export_to_tf_tensor(y))
    out_want, _, _ = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                                    act_dtype, nonpadding=nonpad,
                                    num_microbatches=2, dense=False,
                                    hidden_uniform=hu)
    out_plain, _, _ = O.moe_layer_v1(
        x, w["w_gate"], w["wi"], w["wo"],
        make_hparams(**dict(kw, moe_dropout_rate=0.0))[1], True, act_dtype,
        nonpadding=nonpad, num_microbatches=2, dense=False)
    assert np.abs(out_want - out_plain).max() > 0.05     # units were dropped
    np.testing.assert_allclose(out_got, out_want,
                               **H.value_tolerance(act_dtype))
  tol = H.value_tolerance(act_dtype)
  assert len(compact_calls) == (1 if compact else 0)
  for g_, k in zip(got, ("dx", "dw_gate", "dwi", "dwo")):
    ref = want[k].reshape(g_.shape)
    np.testing.assert_allclose(
        g_, ref, rtol=tol["rtol"], atol=tol["atol"] * max(1.0, np.abs(ref).max()),
        err_msg=k)
  if noise_policy or hidden_dropout:
    return        # a second step would draw new noise
  # a second step re-runs forward and backward on new tokens
  x2 = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype,
                     top=4).reshape(b, l, m)
  lowering.run({xt: torch.from_numpy(x2).to(dt).cuda()})
  want2 = O.moe_layer_v1_backward(x2, w["w_gate"], w["wi"], w["wo"], ohp, True,
                                  act_dtype, d_out, 1.5, nonpadding=nonpad,
                                  num_microbatches=2)
  got2 = H.to_np(lowering.export_to_tf_tensor(grads[2]))
  np.testing.assert_allclose(
      got2, want2["dwi"], rtol=tol["rtol"],
      atol=tol["atol"] * max(1.0, np.abs(want2["dwi"]).max()))


def test_v1_expert_selection_matches_oracle():
  b, l, m, hdim, e, group = 2, 128, 32, 64, 4, 64
  rng = np.random.default_rng(401)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  nonpad = (rng.random((b, l)) < 0.85).astype(np.float32)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_eval=1.0,
                         **dict(SWITCH_HP, moe_gating="expert_selection"))
  # tokens whose router logits keep every expert's ranking unambiguous
  for _ in range(50):
    x = rng.standard_normal((b, l, m)).astype(np.float32)
    logits = O.router_logits(x.reshape(-1, group, m), w["w_gate"])
    ok = True
    for gi in range(logits.shape[0]):
      keep = nonpad.reshape(-1, group)[gi] != 0
      if (np.diff(np.sort(logits[gi][keep], axis=0), axis=0) < 1e-4).any():
        ok = False
    if ok:
      break
  assert ok
  want, want_loss, aux = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                        False, "float32", nonpadding=nonpad)
  wi = dict(w)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpad), mtf.Shape(dims[:2]))
  with mtf.variable_scope("moe"):
    y, loss = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, False, mtf.VariableDType(torch.float32), nonpadding=npad)
  names = sorted(v.name for v in graph.all_variables)
  assert names[0] == "moe/expert_selection_gating/kernel"
  lowering = mtf.Lowering(
      graph, {mesh: mtf.HipMeshImpl()},
      initial_values={"moe/expert_selection_gating/kernel": wi["w_gate"],
                      "moe/wi/kernel": wi["wi"], "moe/wo/kernel": wi["wo"]})
  got = H.to_np(lowering.export_to_tf_tensor(y))
  np.testing.assert_allclose(got, want, **H.value_tolerance("float32"))
  np.testing.assert_allclose(float(H.to_np(lowering.export_to_tf_tensor(loss))),
                             want_loss, rtol=1e-4)
  with pytest.raises(ValueError, match="needs nonpadding"):
    run_v1(x, w, hp, False, "float32")


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_v1_experts_attention(act_dtype):
  """moe_use_experts_attention: two output projections ("q_wo", "k_wo") of the
  same hidden tensor (transformer/moe.py:514-522)."""
  b, l, m, hdim, e, group = 2, 64, 64, 128, 4, 32
  rng = np.random.default_rng(501)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  k_wo = H.normal_weights(rng, (e, hdim, m), hdim)
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype).reshape(b, l, m)
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_use_experts_attention=True)
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  with mtf.variable_scope("moe"):
    outs, loss = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, True, mtf.VariableDType(torch.float32, torch.float32, dt))
  assert isinstance(outs, list) and len(outs) == 2
  assert sorted(v.name for v in graph.all_variables) == [
      "moe/k_wo/kernel", "moe/q_wo/kernel", "moe/top_2_gating/kernel",
      "moe/wi/kernel"]
  lowering = mtf.Lowering(
      graph, {mesh: mtf.HipMeshImpl()},
      initial_values={"moe/top_2_gating/kernel": w["w_gate"],
                      "moe/wi/kernel": w["wi"], "moe/q_wo/kernel": w["wo"],
                      "moe/k_wo/kernel": k_wo})
  q, k = (H.to_np(lowering.export_to_tf_tensor(t)) for t in outs)
  want, want_loss, _ = O.moe_layer_v1(x, w["w_gate"], w["wi"], w["wo"], ohp,
                                      True, act_dtype, dense=False, k_wo=k_wo)
  np.testing.assert_allclose(q, want[0], **H.value_tolerance(act_dtype))
  np.testing.assert_allclose(k, want[1], **H.value_tolerance(act_dtype))
  # each output is bit for bit the plain layer with that output kernel
  hp_plain, _ = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                             moe_group_size=group)
  plain_k, _, _, _ = run_v1(x, dict(w, wo=k_wo), hp_plain, True, act_dtype)
  np.testing.assert_array_equal(k, plain_k)


@pytest.mark.parametrize("case", [
    ("gelu", "float32", "top_2", False, False),
    ("swish", "bfloat16", "switch", False, False),
    (["gelu", "linear"], "float32", "top_2", False, False),
    (["gelu", "linear"], "bfloat16", "top_2", True, False),
    (["tanh", "sigmoid", "relu"], "float32", "switch", True, False),
    (["relu", "linear"], "float32", "top_2", False, True),
    ("sigmoid", "float32", "top_2", True, True),
    ("relu", "float32", "expert_selection", False, False),
    ("relu", "bfloat16", "expert_selection", True, False),
    (["gelu", "linear"], "float32", "expert_selection", False, True)],
    ids=lambda c: "%s-%s-%s%s%s" % ("*".join(c[0]) if isinstance(c[0], list)
                                    else c[0], c[1], c[2],
                                    "-dropout" if c[3] else "",
                                    "-experts_attention" if c[4] else ""))
def test_v1_gradients_other_activations(case):
  """Experts that are not one ReLU / linear layer (other activations, products
  of dense layers), with and without the hidden dropout and the second output
  projection: mtf.gradients against the oracle's backward (pinned by central
  differences in tests/test_oracle.py)."""
  activation, act_dtype, gating, dropout, attention = case
  acts = activation if isinstance(activation, list) else [activation]
  b, l, m, hdim, e, group = 2, 64, 32, 48, 4, 32
  rng = np.random.default_rng(131)
  w_gate = H.normal_weights(rng, (m, e), m)
  wis = [H.normal_weights(rng, (e, m, hdim), m) for _ in acts]
  wo = H.normal_weights(rng, (e, hdim, m), hdim)
  k_wo = H.normal_weights(rng, (e, hdim, m), hdim)
  x = H.safe_tokens(rng, b * l, m, w_gate, act_dtype, top=3).reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.9).astype(np.float32)
  if gating == "expert_selection":
    # tokens whose router logits keep every expert's ranking of the group's
    # tokens unambiguous (the experts choose, per column)
    for _ in range(200):
      x = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
      lg = O.router_logits(x.reshape(-1, group, m), O.cast_act(w_gate, act_dtype))
      gaps = [np.diff(np.sort(lg[gi][nonpad.reshape(-1, group)[gi] != 0], axis=0),
                      axis=0).min() for gi in range(lg.shape[0])]
      if min(gaps) > 1e-4:    # both implementations see the same rounded inputs
        break
    assert min(gaps) > 1e-4
  d_q, d_k = (O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32),
                         act_dtype) for _ in range(2))
  kw = dict(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
            moe_capacity_factor_train=1.0, moe_loss_coef=0.25,
            moe_dropout_rate=0.25 if dropout else 0.0,
            moe_use_experts_attention=attention)
  if gating != "top_2":
    kw.update(SWITCH_HP, moe_gating=gating)
  hp, ohp = make_hparams(**kw)
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  imp = lambda a, shape: mtf.import_tf_tensor(
      mesh, torch.from_numpy(np.asarray(a, np.float32)).to(dt), mtf.Shape(shape))
  xt = imp(x, dims)
  with mtf.variable_scope("moe"):
    outs, loss = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, True, mtf.VariableDType(torch.float32, torch.float32, dt),
        nonpadding=imp(nonpad, dims[:2]), activation=activation,
        num_microbatches=2)
  outs = outs if attention else [outs]
  router = {"switch": "switch_gating",
            "expert_selection": "expert_selection_gating"}.get(
                gating, "top_2_gating")
  wi_names = (["moe/wi_%d/kernel" % i for i in range(len(acts))]
              if len(acts) > 1 else ["moe/wi/kernel"])
  wo_names = (["moe/q_wo/kernel", "moe/k_wo/kernel"] if attention
              else ["moe/wo/kernel"])
  names = ["moe/%s/kernel" % router] + wi_names + wo_names
  values = [w_gate] + wis + ([wo, k_wo] if attention else [wo])
  by_name = {v.name: v.outputs[0] for v in graph.trainable_variables}
  assert sorted(by_name) == sorted(names)
  grads = mtf.gradients(
      outs + [loss], [xt] + [by_name[n] for n in names],
      grad_ys=[imp(d, dims) for d in (d_q, d_k)[:len(outs)]] + [imp(1.5, [])])
  torch.manual_seed(77)
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()},
                          initial_values=dict(zip(names, values)))
  got = dict(zip(["dx"] + names, (H.to_np(lowering.export_to_tf_tensor(g))
                                  for g in grads)))
  hu = None
  if dropout:          # the layer's only random call, reproduced
    torch.manual_seed(77)
    cap = O.expert_capacity(group, 1.0, e, 4)
    hu = torch.rand((e, (b * l // group) * cap, hdim), dtype=dt,
                    device="cuda").float().cpu().numpy()
  wi_arg = wis if len(acts) > 1 else wis[0]
  want = O.moe_layer_v1_backward(
      x, w_gate, wi_arg, wo, ohp, True, act_dtype,
      [d_q, d_k] if attention else d_q, 1.5, nonpadding=nonpad,
      activation=activation, num_microbatches=2, hidden_uniform=hu,
      k_wo=k_wo if attention else None)
  ref = {"dx": want["dx"], names[0]: want["dw_gate"], wo_names[0]: want["dwo"]}
  ref.update(zip(wi_names, want["dwi"] if len(acts) > 1 else [want["dwi"]]))
  if attention:
    ref[wo_names[1]] = want["dk_wo"]
  tol = H.value_tolerance(act_dtype)
  for k, g_ in got.items():
    r_ = ref[k].reshape(g_.shape)
    assert np.abs(r_).max() > 0
    np.testing.assert_allclose(
        g_, r_, rtol=tol["rtol"], atol=tol["atol"] * max(1.0, np.abs(r_).max()),
        err_msg=k)
  # the forward values with the pre-activations kept equal those without
  if not dropout and not attention:
    hp_e = make_hparams(**dict(kw, moe_capacity_factor_eval=1.0))[0]
    fwd = run_v1(x, dict(w_gate=w_gate, wi=wi_arg, wo=wo), hp_e, False,
                 act_dtype, nonpadding=nonpad, activation=activation)[0]
    np.testing.assert_array_equal(
        H.to_np(lowering.export_to_tf_tensor(outs[0])), fwd)


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_v1_experts_attention_gradients(act_dtype):
  """Gradients through both outputs of the layer with
  moe_use_experts_attention: the shared tensors get the sum of the two
  projections' shares."""
  b, l, m, hdim, e, group = 2, 64, 32, 48, 4, 32
  rng = np.random.default_rng(521)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  k_wo = H.normal_weights(rng, (e, hdim, m), hdim)
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], act_dtype).reshape(b, l, m)
  d_q, d_k = (O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32),
                         act_dtype) for _ in range(2))
  hp, ohp = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=group, moe_use_experts_attention=True,
                         moe_capacity_factor_train=1.0, moe_loss_coef=0.25)
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  imp = lambda a, shape: mtf.import_tf_tensor(
      mesh, torch.from_numpy(np.asarray(a, np.float32)).to(dt), mtf.Shape(shape))
  xt = imp(x, dims)
  with mtf.variable_scope("moe"):
    outs, loss = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, True, mtf.VariableDType(torch.float32, torch.float32, dt))
  by_name = {v.name: v.outputs[0] for v in graph.trainable_variables}
  names = ["moe/top_2_gating/kernel", "moe/wi/kernel", "moe/q_wo/kernel",
           "moe/k_wo/kernel"]
  grads = mtf.gradients(outs + [loss], [xt] + [by_name[n] for n in names],
                        grad_ys=[imp(d_q, dims), imp(d_k, dims), imp(1.5, [])])
  lowering = mtf.Lowering(
      graph, {mesh: mtf.HipMeshImpl()},
      initial_values=dict(zip(names, (w["w_gate"], w["wi"], w["wo"], k_wo))))
  got = [H.to_np(lowering.export_to_tf_tensor(g)) for g in grads]
  want = O.moe_layer_v1_backward(x, w["w_gate"], w["wi"], w["wo"], ohp, True,
                                 act_dtype, [d_q, d_k], 1.5, k_wo=k_wo)
  assert not (want["aux"]["kept_1"] & want["aux"]["kept_2"]).all()
  only_q = O.moe_layer_v1_backward(
      x, w["w_gate"], w["wi"], w["wo"],
      make_hparams(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
                   moe_capacity_factor_train=1.0, moe_loss_coef=0.25)[1],
      True, act_dtype, d_q, 1.5)
  assert np.abs(want["dx"] - only_q["dx"]).max() > 0.1   # the k branch matters
  tol = H.value_tolerance(act_dtype)
  for g_, k in zip(got, ("dx", "dw_gate", "dwi", "dwo", "dk_wo")):
    ref = want[k].reshape(g_.shape)
    np.testing.assert_allclose(
        g_, ref, rtol=tol["rtol"], atol=tol["atol"] * max(1.0, np.abs(ref).max()),
        err_msg=k)


@pytest.mark.parametrize("case", [("float32", False), ("bfloat16", False),
                                  ("float32", True)],
                         ids=["float32", "bfloat16", "float32-second_place_loss"])
def test_v2_gradients_match_oracle(case):
  """mtf.gradients over the hierarchical layer against the oracle's backward
  (pinned by central differences in tests/test_oracle.py)."""
  act_dtype, loss2 = case
  b, l, m, hdim, xe, ye, group = 2, 64, 32, 48, 2, 4, 32
  hp, ohp = make_hparams(moe_num_experts=[xe, ye], moe_hidden_size=hdim,
                         moe_group_size=group, moe_capacity_factor_train=1.25,
                         moe_capacity_factor_second_level=1.0,
                         moe_loss_coef=0.25, moe_use_second_place_loss=loss2)
  for seed in range(601, 621):   # first seed without an inner-level near-tie
    rng = np.random.default_rng(seed)
    w = v2_weights(rng, m, hdim, xe, ye)
    x = H.safe_tokens(rng, b * l, m, w["w_outer"], act_dtype).reshape(b, l, m)
    nonpad = (rng.random((b, l)) < 0.9).astype(np.float32)
    _, _, aux = O.moe_layer_v2(x, w["w_outer"], w["w_inner"], w["wi"], w["wo"],
                               ohp, True, act_dtype, nonpadding=nonpad,
                               dense=False)
    if inner_gap_ok(aux):
      break
  assert inner_gap_ok(aux)
  d_out = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpad).to(dt),
                              mtf.Shape(dims[:2]))
  with mtf.variable_scope("moe2d"):
    y, loss = moe.transformer_moe_layer_v2(
        xt, dims[-1], hp, True, mtf.VariableDType(torch.float32, torch.float32, dt),
        nonpadding=npad, num_microbatches=2)
  variables = graph.trainable_variables
  assert [v.name.split("/")[-2] for v in variables] == [
      "outer_gating", "inner_gating", "wi", "wo"]
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(d_out).to(dt), mtf.Shape(dims))
  dlt = mtf.import_tf_tensor(mesh, torch.tensor(1.5, dtype=dt), mtf.Shape([]))
  grads = mtf.gradients([y, loss], [xt] + [v.outputs[0] for v in variables],
                        grad_ys=[dyt, dlt])
  init = {"moe2d/outer_gating/kernel": w["w_outer"],
          "moe2d/inner_gating/kernel": w["w_inner"],
          "moe2d/wi/kernel": w["wi"], "moe2d/wo/kernel": w["wo"]}
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = [H.to_np(lowering.export_to_tf_tensor(g)) for g in grads]
  want = O.moe_layer_v2_backward(x, w["w_outer"], w["w_inner"], w["wi"], w["wo"],
                                 ohp, True, act_dtype, d_out, 1.5,
                                 nonpadding=nonpad, num_microbatches=2)
  tol = H.value_tolerance(act_dtype)
  for g_, k in zip(got, ("dx", "dw_outer", "dw_inner", "dwi", "dwo")):
    ref = want[k].reshape(g_.shape)
    np.testing.assert_allclose(
        g_, ref, rtol=tol["rtol"], atol=tol["atol"] * max(1.0, np.abs(ref).max()),
        err_msg=k)


# ---- random configurations ------------------------------------------------------
def _random_v1_config(rng, gatings, max_tokens):
  """A layer configuration drawn so that the sizes fall on both sides of what
  selects the kernels (matrix-core GEMMs from 256 columns / 128 rows on,
  compacted expert rows when an expert's slot rows are whole 256-row tiles,
  the one-launch router from groups of 128 tokens on)."""
  c = dict(gating=str(rng.choice(gatings)),
           act=str(rng.choice(["float32", "bfloat16"])),
           e=int(rng.choice([2, 4, 5, 8, 16, 32])),
           group=int(rng.choice([32, 64, 128, 256, 512, 1024])),
           m=int(rng.choice([16, 24, 64, 128, 256])),
           hdim=int(rng.choice([40, 64, 128, 256, 512])),
           cf=float(rng.choice([0.5, 1.0, 1.25, 2.0])),
           nonpad=bool(rng.integers(2)), loss2=bool(rng.integers(2)),
           policy=str(rng.choice(["all", "none", "threshold"])))
  c["groups"] = max(1, min(int(rng.integers(1, 5)), max_tokens // c["group"]))
  return c


def _random_v1_inputs(rng, c, top):
  b, l, m, e, hdim = c["groups"], c["group"], c["m"], c["e"], c["hdim"]
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  x = H.safe_tokens(rng, b * l, m, w["w_gate"], c["act"], top=min(top, e),
                    bf16_router=(c["gating"] == "ntlb" and
                                 c["act"] == "bfloat16")).reshape(b, l, m)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32) if c["nonpad"] else None
  kw = dict(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=l,
            moe_capacity_factor_train=c["cf"], moe_capacity_factor_eval=c["cf"],
            moe_loss_coef=0.25)
  if c["gating"] == "top_2":
    kw.update(moe_use_second_place_loss=c["loss2"],
              moe_second_policy_train=c["policy"],
              moe_second_policy_eval=c["policy"],
              moe_second_threshold_train=0.3, moe_second_threshold_eval=0.3)
  else:
    kw.update(SWITCH_HP, moe_gating=c["gating"], moe_ntlb_top_k=min(3, e),
              moe_switch_policy_eval="argmax",
              moe_z_loss=0.1 if c["gating"] == "switch" and c["nonpad"] else None)
  return w, x, nonpad, kw


def test_v1_random_configs_match_oracle():
  """Forward of the layer at 60 random configurations (router, dtype, train /
  eval, sizes, capacity factor, second-place policy and loss, nonpadding)
  against the oracle.  (1500 seeds of this sweep passed when it was written.)"""
  for seed in range(60):
    rng = np.random.default_rng(7000 + seed)
    c = _random_v1_config(rng, ["top_2", "top_2", "switch"], 4096)
    train = bool(rng.integers(2))
    w, x, nonpad, kw = _random_v1_inputs(rng, c, 2)
    hp, ohp = make_hparams(**kw)
    got, got_loss, _, _ = run_v1(x, w, hp, train, c["act"], nonpadding=nonpad,
                                 num_microbatches=2)
    want, want_loss, _ = O.moe_layer_v1(
        x, w["w_gate"], w["wi"], w["wo"], ohp, train, c["act"],
        nonpadding=nonpad, num_microbatches=2, dense=True)
    np.testing.assert_allclose(got, want, err_msg=str((seed, c)),
                               **H.value_tolerance(c["act"]))
    np.testing.assert_allclose(
        got_loss, want_loss, err_msg=str((seed, c)),
        rtol=1e-2 if c["act"] == "bfloat16" else 1e-4)


def test_v1_random_configs_gradients_match_oracle():
  """mtf.gradients of the layer at 60 random configurations against the
  oracle's backward.  The seeds are a fixed range in which no hidden unit's
  pre-activation sits at the ReLU kink: 3 of 1350 seeds of this sweep had one
  token whose d(tokens) row differed because one pre-activation was +3.5e-8 in
  float64 and -6.5e-9 as a float32 sum, so the two sides disagreed on that
  unit's ReLU derivative (checked for each of the three; every other seed
  passed)."""
  for seed in range(60):
    rng = np.random.default_rng(8000 + seed)
    c = _random_v1_config(rng, ["top_2", "top_2", "switch", "ntlb"], 2048)
    b, l, m = c["groups"], c["group"], c["m"]
    w, x, nonpad, kw = _random_v1_inputs(rng, c, 4)
    d_out = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), c["act"])
    hp, ohp = make_hparams(**kw)
    dt = H.ACT_TORCH[c["act"]]
    graph = mtf.Graph()
    mesh = mtf.Mesh(graph, "mesh")
    dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
            mtf.Dimension("d_model", m)]
    xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
    npad = None
    if nonpad is not None:
      npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpad).to(dt),
                                  mtf.Shape(dims[:2]))
    with mtf.variable_scope("moe"):
      y, loss = moe.transformer_moe_layer_v1(
          xt, dims[-1], hp, True,
          mtf.VariableDType(torch.float32, torch.float32, dt), nonpadding=npad,
          num_microbatches=2)
    variables = graph.trainable_variables
    dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(d_out).to(dt),
                               mtf.Shape(dims))
    dlt = mtf.import_tf_tensor(mesh, torch.tensor(1.5, dtype=dt), mtf.Shape([]))
    grads = mtf.gradients([y, loss], [xt] + [v.outputs[0] for v in variables],
                          grad_ys=[dyt, dlt])
    router = {"switch": "switch_gating", "ntlb": "ntlb_gating"}.get(
        c["gating"], "top_2_gating")
    lowering = mtf.Lowering(
        graph, {mesh: mtf.HipMeshImpl()},
        initial_values={"moe/%s/kernel" % router: w["w_gate"],
                        "moe/wi/kernel": w["wi"], "moe/wo/kernel": w["wo"]})
    got = [H.to_np(lowering.export_to_tf_tensor(g)) for g in grads]
    want = O.moe_layer_v1_backward(
        x, w["w_gate"], w["wi"], w["wo"], ohp, True, c["act"], d_out, 1.5,
        nonpadding=nonpad, num_microbatches=2)
    tol = H.value_tolerance(c["act"])
    for g_, k in zip(got, ("dx", "dw_gate", "dwi", "dwo")):
      ref = want[k].reshape(g_.shape)
      np.testing.assert_allclose(
          g_, ref, rtol=tol["rtol"],
          atol=tol["atol"] * max(1.0, np.abs(ref).max()),
          err_msg=str((k, seed, c)))


def test_v2_random_configs_match_oracle():
  """Forward and gradients of the hierarchical layer at 40 random
  configurations (expert grid, group size, both capacity factors, sizes, dtype,
  nonpadding, second-place loss) against the oracle.  (1700 forward and 600
  gradient seeds of this sweep passed when it was written.)"""
  for seed in range(40):
    rng = np.random.default_rng(9000 + seed)
    act = str(rng.choice(["float32", "bfloat16"]))
    xe, ye = int(rng.choice([2, 3, 4, 8])), int(rng.choice([2, 4, 5, 8]))
    group = int(rng.choice([32, 64, 128, 256, 512]))
    m, hdim = int(rng.choice([16, 32, 64, 128])), int(rng.choice([32, 48, 128, 256]))
    cf, cf2 = float(rng.choice([1.0, 1.25, 2.0])), float(rng.choice([0.5, 1.0, 1.5]))
    b, l = max(1, min(int(rng.integers(1, 5)), 2048 // group)), group
    loss2, use_np = bool(rng.integers(2)), bool(rng.integers(2))
    case = dict(seed=seed, act=act, xe=xe, ye=ye, group=group, b=b, m=m,
                hdim=hdim, cf=cf, cf2=cf2, loss2=loss2, nonpad=use_np)
    hp, ohp = make_hparams(
        moe_num_experts=[xe, ye], moe_hidden_size=hdim, moe_group_size=group,
        moe_capacity_factor_train=cf, moe_capacity_factor_second_level=cf2,
        moe_loss_coef=0.25, moe_use_second_place_loss=loss2)
    for _ in range(20):            # weights and tokens without inner near-ties
      w = v2_weights(rng, m, hdim, xe, ye)
      x = H.safe_tokens(rng, b * l, m, w["w_outer"], act)
      x = safe_tokens_v2(rng, x, w, act).reshape(b, l, m)
      nonpad = (rng.random((b, l)) < 0.9).astype(np.float32) if use_np else None
      fwd, fwd_loss, aux = O.moe_layer_v2(
          x, w["w_outer"], w["w_inner"], w["wi"], w["wo"], ohp, True, act,
          nonpadding=nonpad, num_microbatches=2, dense=False)
      if inner_gap_ok(aux):
        break
    assert inner_gap_ok(aux), case
    d_out = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act)
    dt = H.ACT_TORCH[act]
    graph = mtf.Graph()
    mesh = mtf.Mesh(graph, "mesh")
    dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
            mtf.Dimension("d_model", m)]
    xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
    npad = None
    if use_np:
      npad = mtf.import_tf_tensor(mesh, torch.from_numpy(nonpad).to(dt),
                                  mtf.Shape(dims[:2]))
    with mtf.variable_scope("moe2d"):
      y, loss = moe.transformer_moe_layer_v2(
          xt, dims[-1], hp, True,
          mtf.VariableDType(torch.float32, torch.float32, dt), nonpadding=npad,
          num_microbatches=2)
    variables = graph.trainable_variables
    dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(d_out).to(dt),
                               mtf.Shape(dims))
    dlt = mtf.import_tf_tensor(mesh, torch.tensor(1.5, dtype=dt), mtf.Shape([]))
    grads = mtf.gradients([y, loss], [xt] + [v.outputs[0] for v in variables],
                          grad_ys=[dyt, dlt])
    lowering = mtf.Lowering(
        graph, {mesh: mtf.HipMeshImpl()},
        initial_values={"moe2d/outer_gating/kernel": w["w_outer"],
                        "moe2d/inner_gating/kernel": w["w_inner"],
                        "moe2d/wi/kernel": w["wi"], "moe2d/wo/kernel": w["wo"]})
    tol = H.value_tolerance(act)
    np.testing.assert_allclose(H.to_np(lowering.export_to_tf_tensor(y)), fwd,
                               err_msg=str(case), **tol)
    np.testing.assert_allclose(
        float(H.to_np(lowering.export_to_tf_tensor(loss))), fwd_loss,
        rtol=1e-2 if act == "bfloat16" else 1e-4, err_msg=str(case))
    got = [H.to_np(lowering.export_to_tf_tensor(g)) for g in grads]
    want = O.moe_layer_v2_backward(
        x, w["w_outer"], w["w_inner"], w["wi"], w["wo"], ohp, True, act, d_out,
        1.5, nonpadding=nonpad, num_microbatches=2)
    for g_, k in zip(got, ("dx", "dw_outer", "dw_inner", "dwi", "dwo")):
      ref = want[k].reshape(g_.shape)
      np.testing.assert_allclose(
          g_, ref, rtol=tol["rtol"],
          atol=tol["atol"] * max(1.0, np.abs(ref).max()),
          err_msg=str((k, case)))


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_captured_step_replays_match_eager(act_dtype):
  """Lowering.capture(): a HIP-graph replay gives what an eager run gives, on
  new tokens, several times, with eager work on the same lowering and
  synchronisations between the replays."""
  b, l, m, hdim, e, group = 2, 256, 64, 128, 8, 128
  rng = np.random.default_rng(501)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  hp, _ = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                       moe_group_size=group)
  dt = H.ACT_TORCH[act_dtype]
  xs = [O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
        for _ in range(4)]
  _, _, lowering, (xt, y) = run_v1(xs[0], w, hp, False, act_dtype)
  step = lowering.capture()
  for i in (1, 2, 3, 1):
    xv = torch.from_numpy(xs[i]).to(dt).cuda()
    lowering.run({xt: xv})                                   # eager
    eager = lowering.export_to_tf_tensor(y).clone()
    torch.cuda.synchronize()
    step.replay({xt: xv})                                    # recorded
    torch.cuda.synchronize()
    assert torch.equal(lowering.export_to_tf_tensor(y), eager), i
  # a replay without feeds repeats the last tokens
  step.replay()
  assert torch.equal(lowering.export_to_tf_tensor(y), eager)
  # new weights between two replays (an optimizer step, a checkpoint restore):
  # the variable's slice and its packed copies are updated in place, so the
  # recorded kernels read the new values
  var = {v.name: lv for v, lv in lowering.variables.items()}
  for trial in range(2):
    var["moe/wi/kernel"].assign(H.normal_weights(rng, (e, m, hdim), m))
    var["moe/top_2_gating/kernel"].assign(H.normal_weights(rng, (m, e), m))
    var["moe/wo/kernel"].assign_to_slices(
        None, [torch.from_numpy(H.normal_weights(rng, (e, hdim, m), hdim)).cuda()])
    torch.cuda.synchronize()
    step.replay()
    torch.cuda.synchronize()
    replayed = lowering.export_to_tf_tensor(y).clone()
    lowering.run({xt: xv})
    assert torch.equal(lowering.export_to_tf_tensor(y), replayed), trial
    assert not torch.equal(replayed, eager)
    eager = replayed


def test_captured_gradient_step_on_compacted_rows():
  """A recorded forward + backward step of a switch layer at a shape whose
  gradient graph stays on compacted rows: every replay, on new tokens, with
  eager steps and synchronisations between the replays, gives what the eager
  step gives.  (The router kernel's gradient is summed with float atomics: it
  is compared to rounding, everything else bit for bit.)"""
  b, l, m, hdim, e, group = 2, 1024, 256, 512, 4, 1024
  rng = np.random.default_rng(611)
  w = dict(w_gate=H.normal_weights(rng, (m, e), m),
           wi=H.normal_weights(rng, (e, m, hdim), m),
           wo=H.normal_weights(rng, (e, hdim, m), hdim))
  hp, _ = make_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                       moe_group_size=group, moe_capacity_factor_train=1.25,
                       **SWITCH_HP)
  dt = torch.bfloat16
  xs = [O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), "bfloat16")
        for _ in range(3)]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(xs[0]).to(dt), mtf.Shape(dims))
  with mtf.variable_scope("moe"):
    y, loss = moe.transformer_moe_layer_v1(
        xt, dims[-1], hp, True, mtf.VariableDType(torch.float32, torch.float32, dt))
  variables = graph.trainable_variables
  d_out = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), "bfloat16")
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(d_out).to(dt), mtf.Shape(dims))
  grads = mtf.gradients([y, loss], [xt] + [v.outputs[0] for v in variables],
                        grad_ys=[dyt, None])
  init = {"moe/switch_gating/kernel": w["w_gate"], "moe/wi/kernel": w["wi"],
          "moe/wo/kernel": w["wo"]}
  from mesh_amd import moe_hip
  with moe_hip.StageTimer() as timer:
    lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  assert timer.compacted == 1
  step = lowering.capture()
  for i in (1, 2, 0, 1):
    xv = torch.from_numpy(xs[i]).to(dt).cuda()
    lowering.run({xt: xv})
    eager = [lowering.export_to_tf_tensor(t).clone() for t in [y] + grads]
    torch.cuda.synchronize()
    step.replay({xt: xv})
    torch.cuda.synchronize()
    for j, (t, want) in enumerate(zip([y] + grads, eager)):
      got = lowering.export_to_tf_tensor(t)
      if j == 2:          # the router kernel's gradient
        np.testing.assert_allclose(
            H.to_np(got), H.to_np(want), rtol=2e-2,
            atol=1e-2 * float(want.float().abs().max()))
      else:
        assert torch.equal(got, want), (i, j)
