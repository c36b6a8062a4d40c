"""Pins the CPU oracle (the reference holds no golden vectors for its MoE file):
each function is checked against brute force, closed forms, float64 library
routines or hand-worked cases, chosen so that a dropped term, a wrong index or a
transposed operand fails."""

import json
import os

import numpy as np
import pytest
import scipy.special

from oracle import moe_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---- host integer logic ------------------------------------------------------
def test_split_into_groups_brute_force():
  """Defining constraints of transformer/moe.py:1555-1557: group_size is the
  largest divisor arrangement with group_size <= max and num_groups a multiple
  of mesh_dim_size (when n allows)."""
  for n in list(range(1, 200)) + [1024, 2048, 4096, 5120, 65536]:
    for max_group in (1, 3, 16, 100, 1024, 2048):
      for mesh in (1, 2, 4, 8):
        if n % mesh:
          with pytest.raises(ValueError):
            O.split_into_groups(n, max_group, mesh)
          continue
        g, s = O.split_into_groups(n, max_group, mesh)
        assert g * s == n and g % mesh == 0
        # brute force: smallest admissible num_groups >= max(1, n // max_group)
        want = next(k for k in range(max(1, n // max_group), n + 1)
                    if k % mesh == 0 and n % k == 0)
        assert g == want
        if n % max_group == 0 and (n // max_group) % mesh == 0:
          assert s == max_group


def test_capacity_table():
  """The five benchmark configurations (S, cf, E, min=4) -> C."""
  assert O.expert_capacity(1024, 1.25, 8, 4) == 160
  assert O.expert_capacity(1024, 1.25, 32, 4) == 40
  assert O.expert_capacity(2048, 1.0, 64, 4) == 32
  assert O.expert_capacity(2048, 2.0, 64, 4) == 64
  assert O.expert_capacity(1024, 1.25, 16, 4) == 80
  assert O.expert_capacity(1024, 1.0, 16, 4) == 64
  assert O.expert_capacity(8, 1.0, 64, 4) == 4       # floor at min capacity
  assert O.expert_capacity(16, 100.0, 2, 4) == 16    # never above group size
  assert O.split_into_groups(8 * 32 * 160 // 8, 1024, 1) == (5, 1024)


# ---- float primitives --------------------------------------------------------
def test_round_bf16_matches_torch():
  import torch
  rng = np.random.default_rng(0)
  a = np.concatenate([
      rng.standard_normal(10000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 10000),
      np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, np.inf, -np.inf,
                3.3895e38, 1e-45], np.float32)])
  want = torch.from_numpy(a).to(torch.bfloat16).float().numpy()
  np.testing.assert_array_equal(O.round_bf16(a), want)
  assert np.isnan(O.round_bf16(np.float32(np.nan)))


def test_softmax_against_float64():
  rng = np.random.default_rng(1)
  x = (rng.standard_normal((50, 7, 33)) * 4).astype(np.float32)
  p = O.softmax(x)
  want = scipy.special.softmax(x.astype(np.float64), axis=-1)
  np.testing.assert_allclose(p, want, rtol=2e-6)
  np.testing.assert_allclose(p.sum(-1), 1.0, atol=1e-6)
  # equal logits -> equal gates, whatever exp/log round to
  eq = O.softmax(np.full((3, 8), 1.7, np.float32))
  assert (eq == eq[:, :1]).all()
  # large offsets do not overflow
  assert np.isfinite(O.softmax(x + np.float32(1e4))).all()


def test_seq_sum_is_sequential():
  a = np.array([1e8, 1.0, -1e8, 1.0], np.float32)
  assert O.seq_sum(a) == np.float32(1.0)     # ((1e8 + 1) - 1e8) + 1 in float32
  rng = np.random.default_rng(2)
  x = rng.standard_normal((4, 9)).astype(np.float32)
  want = np.zeros(4, np.float32)
  for j in range(9):
    want = want + x[:, j]
  np.testing.assert_array_equal(O.seq_sum(x), want)


def test_cumsum_dense_equals_index_form():
  rng = np.random.default_rng(3)
  x = (rng.random((3, 40, 6)) < 0.3).astype(np.float32)
  a, b = O.cumsum_exclusive(x, dense=True), O.cumsum_exclusive(x)
  np.testing.assert_array_equal(a, b)
  assert (a[:, 0] == 0).all()
  np.testing.assert_array_equal(a[:, 1:], np.cumsum(x, axis=1)[:, :-1])


# ---- top-2 selection -----------------------------------------------------------
def test_top2_against_stable_argsort():
  rng = np.random.default_rng(4)
  logits = rng.standard_normal((5, 64, 12)).astype(np.float32)
  r = O.top_2_gating(logits, 1000)
  p = O.softmax(logits)
  order = np.argsort(-p, axis=-1, kind="stable")
  np.testing.assert_array_equal(r["index_1"], order[..., 0])
  np.testing.assert_array_equal(r["index_2"], order[..., 1])
  g1 = np.take_along_axis(p, order[..., :1], -1)[..., 0]
  g2 = np.take_along_axis(p, order[..., 1:2], -1)[..., 0]
  np.testing.assert_allclose(r["gate_1"], g1 / (g1 + g2 + 1e-9), rtol=1e-6)
  np.testing.assert_allclose(r["gate_1"] + r["gate_2"], 1.0, atol=1e-6)


def test_top2_exact_ties_lowest_index_wins():
  logits = np.zeros((1, 4, 5), np.float32)
  logits[0, 1, [2, 4]] = 1.0          # two-way tie for first
  logits[0, 2, 3] = 2.0               # clear first, four-way tie for second
  r = O.top_2_gating(logits, 100)
  np.testing.assert_array_equal(r["index_1"][0], [0, 2, 3, 0])
  np.testing.assert_array_equal(r["index_2"][0], [1, 4, 0, 1])


def test_two_experts_always_both():
  rng = np.random.default_rng(5)
  r = O.top_2_gating(rng.standard_normal((2, 30, 2)).astype(np.float32), 100)
  assert (r["index_1"] != r["index_2"]).all()
  assert r["kept_1"].all() and r["kept_2"].all()


# ---- capacity positions --------------------------------------------------------
def test_hand_worked_capacity_case():
  """One group, S=6, E=3, C=2; worked by hand from transformer/moe.py:1472-1496."""
  big, mid = 5.0, 3.0
  idx1 = [0, 0, 1, 0, 2, 1]
  idx2 = [1, 2, 0, 1, 0, 0]
  logits = np.zeros((1, 6, 3), np.float32)
  for s, (a, b) in enumerate(zip(idx1, idx2)):
    logits[0, s, a], logits[0, s, b] = big, mid
  r = O.top_2_gating(logits, 2)
  np.testing.assert_array_equal(r["index_1"][0], idx1)
  np.testing.assert_array_equal(r["index_2"][0], idx2)
  np.testing.assert_array_equal(r["pos_1"][0], [0, 1, 0, 2, 0, 1])
  np.testing.assert_array_equal(r["kept_1"][0], [1, 1, 1, 0, 1, 1])
  np.testing.assert_array_equal(r["pos_2"][0], [2, 1, 2, 3, 3, 4])
  np.testing.assert_array_equal(r["kept_2"][0], [0, 1, 0, 0, 0, 0])
  np.testing.assert_array_equal(r["fill"][0], [2, 2, 2])
  # token 3 lost both choices; token 0 keeps its un-renormalised first gate
  assert r["gate_1"][0, 3] == 0 and r["gate_2"][0, 3] == 0
  p = O.softmax(logits)[0, 0]
  np.testing.assert_allclose(r["gate_1"][0, 0], p[0] / (p[0] + p[1] + 1e-9),
                             rtol=1e-6)


@pytest.mark.parametrize("seed", range(6))
def test_capacity_against_sequential_loop(seed):
  rng = np.random.default_rng(100 + seed)
  g, s, e = 3, int(rng.integers(5, 90)), int(rng.integers(2, 9))
  c = int(rng.integers(1, 2 * s // e + 2))
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  imp = None
  if seed % 2:
    imp = rng.choice(np.array([0.0, 0.5, 1.0], np.float32), size=(g, s))
  for dense in (False, True):
    r = O.top_2_gating(logits, c, importance=imp, dense=dense)
    sel1 = np.ones((g, s), bool) if imp is None else imp == 1.0
    sel2 = np.ones((g, s), bool) if imp is None else imp > 0
    p1, k1, p2, k2, fill = O.routing_sequential(r["index_1"], r["index_2"],
                                                sel1, sel2, e, c)
    np.testing.assert_array_equal(r["kept_1"], k1)
    np.testing.assert_array_equal(r["kept_2"], k2)
    np.testing.assert_array_equal(r["pos_1"], p1)
    np.testing.assert_array_equal(r["pos_2"], p2)
    np.testing.assert_array_equal(r["fill"], fill)


def test_capacity_invariants():
  rng = np.random.default_rng(7)
  g, s, e, c = 4, 200, 8, 30
  r = O.top_2_gating(rng.standard_normal((g, s, e)).astype(np.float32), c)
  for gi in range(g):
    for ex in range(e):
      pos = np.concatenate([
          r["pos_1"][gi][(r["index_1"][gi] == ex) & r["kept_1"][gi]],
          r["pos_2"][gi][(r["index_2"][gi] == ex) & r["kept_2"][gi]]])
      assert sorted(pos.tolist()) == list(range(len(pos))) and len(pos) <= c
      assert len(pos) == r["fill"][gi, ex]
      first = r["pos_1"][gi][(r["index_1"][gi] == ex) & r["kept_1"][gi]]
      assert (np.diff(first) > 0).all()
  # nothing is dropped when capacity covers both choices of every token
  r = O.top_2_gating(rng.standard_normal((g, s, e)).astype(np.float32), 2 * s)
  assert r["kept_1"].all() and r["kept_2"].all()
  # all tokens to one expert: exactly the first C survive
  one = np.zeros((1, 50, 4), np.float32)
  one[..., 2] = 5.0
  r = O.top_2_gating(one, 7)
  np.testing.assert_array_equal(r["kept_1"][0], np.arange(50) < 7)


def test_importance_semantics():
  """importance 1 -> up to two experts; 0 < importance < 1 -> best expert only,
  at second priority, gate ~ 1; importance 0 -> nowhere
  (transformer/moe.py:1347-1355, :1401-1411)."""
  rng = np.random.default_rng(8)
  logits = rng.standard_normal((1, 9, 4)).astype(np.float32)
  imp = np.array([[1, 0.5, 0, 1, 0.5, 0.3, 1, 0, 1]], np.float32)
  r = O.top_2_gating(logits, 100, importance=imp)
  half = (imp > 0) & (imp < 1)
  assert (r["index_2"][half] == r["index_1"][half]).all()
  assert not r["kept_1"][half].any() and r["kept_2"][half].all()
  np.testing.assert_allclose(r["gate_2"][half], 1.0, atol=1e-6)
  assert not r["kept_1"][imp == 0].any() and not r["kept_2"][imp == 0].any()
  assert r["kept_1"][imp == 1].all() and r["kept_2"][imp == 1].all()


def test_second_policies():
  rng = np.random.default_rng(9)
  logits = rng.standard_normal((2, 60, 6)).astype(np.float32)
  base = O.top_2_gating(logits, 1000)
  none = O.top_2_gating(logits, 1000, policy="none")
  assert not none["kept_2"].any() and none["kept_1"].all()
  thr = O.top_2_gating(logits, 1000, policy="threshold", threshold=0.3)
  np.testing.assert_array_equal(thr["kept_2"], base["gate_2"] > np.float32(0.3))
  u = rng.random((2, 60)).astype(np.float32)
  rnd = O.top_2_gating(logits, 1000, policy="random", threshold=0.25,
                       second_uniform=u)
  np.testing.assert_array_equal(rnd["kept_2"],
                                u < base["gate_2"] * np.float32(4.0))
  with pytest.raises(ValueError):
    O.top_2_gating(logits, 10, policy="sometimes")


# ---- dense tensors, dispatch, combine -----------------------------------------
@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_dense_tensors_match_index_record(act_dtype):
  rng = np.random.default_rng(10)
  g, s, e, c, m = 2, 40, 5, 9, 8
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  r = O.top_2_gating(logits, c, act_dtype=act_dtype, dense=True)
  w1, w2 = O.combine_weights(r, act_dtype)
  rebuilt = np.zeros((g, s, e, c), np.float32)
  for gi in range(g):
    for si in range(s):
      if r["kept_1"][gi, si]:
        rebuilt[gi, si, r["index_1"][gi, si], r["pos_1"][gi, si]] += w1[gi, si]
      if r["kept_2"][gi, si]:
        rebuilt[gi, si, r["index_2"][gi, si], r["pos_2"][gi, si]] += w2[gi, si]
  np.testing.assert_array_equal(r["combine"], rebuilt)
  np.testing.assert_array_equal(r["dispatch"], (rebuilt != 0).astype(np.float32))
  assert (r["dispatch"].sum(axis=1) <= 1).all()         # one token per slot
  x = O.cast_act(rng.standard_normal((g, s, m)).astype(np.float32), act_dtype)
  np.testing.assert_array_equal(
      O.dispatch_gather(x, r, e, c, act_dtype),
      np.einsum("gsm,gsec->egcm", x, r["dispatch"]).astype(np.float32))
  y = O.cast_act(rng.standard_normal((e, g, c, m)).astype(np.float32), act_dtype)
  dense_out = np.einsum("egcn,gsec->gsn", y.astype(np.float64),
                        r["combine"].astype(np.float64))
  got = O.combine_gather(y, r, act_dtype)
  tol = 1e-2 if act_dtype == "bfloat16" else 1e-6
  np.testing.assert_allclose(got, dense_out, rtol=tol, atol=tol)


def test_expert_ffn_against_float64():
  rng = np.random.default_rng(11)
  e, rows, m, h, n = 3, 17, 12, 20, 10
  x = rng.standard_normal((e, rows, m)).astype(np.float32)
  wi = rng.standard_normal((e, m, h)).astype(np.float32)
  wo = rng.standard_normal((e, h, n)).astype(np.float32)
  got = O.expert_ffn(x, wi, wo, "relu", "float32")
  want = np.zeros((e, rows, n))
  for k in range(e):   # explicit per-expert loops: a transposed operand fails
    hid = np.maximum(x[k].astype(np.float64) @ wi[k].astype(np.float64), 0)
    want[k] = hid @ wo[k].astype(np.float64)
  np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
  lin = O.expert_ffn(x, wi, wo, "linear", "float32")
  assert not np.allclose(lin, got)


def test_balanced_routing_loss_is_one():
  """Perfectly balanced first choices with uniform gates: density = proxy = 1/E,
  loss = mean(1/E^2) * E^2 = 1 (transformer/moe.py:1420-1424)."""
  e, s = 8, 64
  logits = np.zeros((2, s, e), np.float32)
  r = O.top_2_gating(logits, 1000)
  # uniform gates but argmax always 0 -> density_1 = [1,0,..]: loss = 1/E * E = 1
  np.testing.assert_allclose(r["loss"], 1.0, rtol=1e-6)
  # truly balanced: token s prefers expert s % E by a hair (gates ~uniform)
  logits[:, np.arange(s), np.arange(s) % e] = 1e-4
  r = O.top_2_gating(logits, 1000)
  np.testing.assert_allclose(r["loss"], 1.0, rtol=1e-4)
  # all mass on one expert: density = proxy = 1 for it -> loss = E
  logits = np.zeros((1, s, e), np.float32)
  logits[..., 3] = 30.0
  np.testing.assert_allclose(O.top_2_gating(logits, 1000)["loss"], e, rtol=1e-5)
  # microbatches divide, the second-place loss adds half of a second term
  a = O.top_2_gating(logits, 1000, num_microbatches=4)["loss"]
  np.testing.assert_allclose(a, e / 4, rtol=1e-5)


def test_second_place_loss_forward_value():
  """moe_use_second_place_loss (transformer/moe.py:1426-1438): a case worked by
  hand, then random logits against a float64 computation written from the
  formulas, with importance and microbatches.

  Hand case, one group, S = 2, E = 3: token 0 has probabilities (.5, .3, .2) ->
  first choice 0, second 1, renormalised remainder (0, .6, .4); token 1 has
  (.2, .2, .6) -> first 2, second 0 (lowest index of the tie), remainder
  (.5, .5, 0).  density_1 = (.5, 0, .5), proxy_1 = (.35, .25, .4): loss_1 =
  (.175 + 0 + .2) / 3 * 9 = 1.125.  density_2 = (.5, .5, 0), proxy_2 =
  (.25, .55, .2): loss_2 = (.125 + .275 + 0) / 3 * 9 = 1.2.  Total 1.125 +
  0.5 * 1.2 = 1.725."""
  p = np.array([[[0.5, 0.3, 0.2], [0.2, 0.2, 0.6]]])
  logits = np.log(p).astype(np.float32)
  r = O.top_2_gating(logits, 4, use_second_place_loss=True)
  assert r["index_1"].tolist() == [[0, 2]] and r["index_2"].tolist() == [[1, 0]]
  np.testing.assert_allclose(r["loss"], 1.725, rtol=1e-6)
  np.testing.assert_allclose(O.top_2_gating(logits, 4)["loss"], 1.125, rtol=1e-6)
  # the policy comes after the loss: it does not change it (moe.py:1444-1467)
  r = O.top_2_gating(logits, 4, use_second_place_loss=True, policy="none")
  np.testing.assert_allclose(r["loss"], 1.725, rtol=1e-6)

  rng = np.random.default_rng(77)
  g, s, e, mb = 3, 40, 6, 4
  logits = rng.standard_normal((g, s, e)).astype(np.float32) * 1.5
  imp = rng.choice(np.array([0.0, 0.5, 1.0], np.float32), size=(g, s))
  got = O.top_2_gating(logits, 5, importance=imp, use_second_place_loss=True,
                       num_microbatches=mb)
  pr = scipy.special.softmax(logits.astype(np.float64), axis=-1)
  one = (imp == 1.0)[..., None]
  eye = np.eye(e)
  mask_1 = eye[pr.argmax(-1)] * one
  q = pr * (1.0 - mask_1)
  mask_2 = eye[q.argmax(-1)] * (imp > 0)[..., None]
  loss_1 = ((pr * one).mean(1) * mask_1.mean(1)).mean() * e * e
  norm = q / (q.sum(-1, keepdims=True) + 1e-9)
  loss_2 = (norm.mean(1) * mask_2.mean(1)).mean() * e * e
  np.testing.assert_allclose(got["loss"], (loss_1 + 0.5 * loss_2) / mb,
                             rtol=2e-6)
  assert loss_2 > 0.1 * loss_1              # the second term is not negligible


# ---- switch (top-1) gating ------------------------------------------------------
@pytest.mark.parametrize("seed", range(4))
def test_switch_against_sequential_loop_and_float64(seed):
  """One choice per token: positions/drops against a per-token integer loop
  written from transformer/moe.py:1268-1291, the gate against a float64 softmax
  (raw probability of the arg-max expert, not normalised)."""
  rng = np.random.default_rng(300 + seed)
  g, s, e = 3, int(rng.integers(5, 90)), int(rng.integers(2, 9))
  c = int(rng.integers(1, s // e + 3))
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  imp = None
  if seed % 2:
    imp = rng.choice(np.array([0.0, 0.5, 1.0], np.float32), size=(g, s))
  p64 = scipy.special.softmax(logits.astype(np.float64), axis=-1)
  for dense in (False, True):
    r = O.switch_gating(logits, c, importance=imp, dense=dense)
    np.testing.assert_array_equal(r["index_1"], p64.argmax(-1))
    assert not r["kept_2"].any() and not r["gate_2"].any()
    for gi in range(g):
      count = [0] * e
      for si in range(s):
        ex = int(r["index_1"][gi, si])
        competes = imp is None or imp[gi, si] == 1.0
        if not competes:
          assert not r["kept_1"][gi, si] and r["gate_1"][gi, si] == 0
          continue
        slot = count[ex]
        count[ex] += 1
        assert r["pos_1"][gi, si] == slot
        assert r["kept_1"][gi, si] == (slot < c)
        want = p64[gi, si, ex] if slot < c else 0.0
        np.testing.assert_allclose(r["gate_1"][gi, si], want, rtol=2e-6)
      np.testing.assert_array_equal(r["fill"][gi], np.minimum(count, c))


def test_switch_first_choice_equals_top2_first_choice():
  """The first-choice bookkeeping of the two routers is the same code path in
  the reference (moe.py:1268-1275 vs :1472-1476): same experts, positions and
  drops; only the gate differs (raw probability vs normalised pair)."""
  rng = np.random.default_rng(31)
  logits = rng.standard_normal((2, 120, 6)).astype(np.float32)
  imp = rng.choice(np.array([0.0, 1.0], np.float32), size=(2, 120))
  a = O.switch_gating(logits, 17, importance=imp)
  b = O.top_2_gating(logits, 17, importance=imp, policy="none")
  for k in ("index_1", "kept_1", "fill"):
    np.testing.assert_array_equal(a[k], b[k])
  np.testing.assert_array_equal(a["pos_1"][a["kept_1"]], b["pos_1"][b["kept_1"]])
  p = O.softmax(logits)
  np.testing.assert_array_equal(a["gate_1"][a["kept_1"]],
                                p.max(-1)[a["kept_1"]])


def test_switch_loss_closed_forms():
  """density_1 is taken before the importance mask and the proxy is multiplied
  by (importance == 1) per token (moe.py:1224-1234): with uniform gates and
  balanced arg-max the loss is the fraction of tokens with importance 1."""
  e, s = 8, 64
  logits = np.zeros((2, s, e), np.float32)
  logits[:, np.arange(s), np.arange(s) % e] = 1e-4
  np.testing.assert_allclose(O.switch_gating(logits, 1000)["loss"], 1.0,
                             rtol=1e-4)
  imp = np.ones((2, s), np.float32)
  imp[0, :16] = 0.0
  imp[1, :32] = 0.5
  r = O.switch_gating(logits, 1000, importance=imp)
  np.testing.assert_allclose(r["loss"], (48 + 32) / 128.0, rtol=1e-4)
  # all mass on one expert -> E; microbatches divide
  one = np.zeros((1, s, e), np.float32)
  one[..., 3] = 30.0
  np.testing.assert_allclose(O.switch_gating(one, 1000)["loss"], e, rtol=1e-5)
  np.testing.assert_allclose(
      O.switch_gating(one, 1000, num_microbatches=4)["loss"], e / 4, rtol=1e-5)


def test_switch_z_loss_closed_form():
  """Constant logits c: logsumexp = c + log E for every token, so
  z_loss = (c + log E)^2 / num_microbatches whatever the mask
  (moe.py:1253-1266); added only when training."""
  e, s, c0 = 4, 32, 1.5
  logits = np.full((2, s, e), c0, np.float32)
  imp = np.ones((2, s), np.float32)
  imp[1, ::3] = 0.0
  base = O.switch_gating(logits, 100, importance=imp, train=True,
                         num_microbatches=2)["loss"]
  got = O.switch_gating(logits, 100, importance=imp, train=True, z_loss=0.1,
                        num_microbatches=2)["loss"]
  np.testing.assert_allclose(got - base, 0.1 * (c0 + np.log(e)) ** 2 / 2,
                             rtol=1e-5)
  evalv = O.switch_gating(logits, 100, importance=imp, train=False, z_loss=0.1,
                          num_microbatches=2)["loss"]
  assert evalv == base
  # masked tokens do not contribute: give them huge logits
  big = logits.copy()
  big[1, ::3] = 40.0
  got2 = O.switch_gating(big, 100, importance=imp, train=True, z_loss=0.1,
                         num_microbatches=2)
  base2 = O.switch_gating(big, 100, importance=imp, train=True,
                          num_microbatches=2)
  np.testing.assert_allclose(got2["loss"] - base2["loss"],
                             0.1 * (c0 + np.log(e)) ** 2 / 2, rtol=1e-4)
  with pytest.raises(ValueError):
    O.switch_gating(logits, 100, train=True, z_loss=0.1, num_microbatches=2)


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_switch_dense_tensors_match_index_record(act_dtype):
  rng = np.random.default_rng(33)
  g, s, e, c = 2, 40, 5, 6
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  r = O.switch_gating(logits, c, act_dtype=act_dtype, dense=True)
  want = np.zeros((g, s, e, c), np.float32)
  w = O.cast_act(r["gate_1"], act_dtype)
  for gi in range(g):
    for si in range(s):
      if r["kept_1"][gi, si]:
        want[gi, si, r["index_1"][gi, si], r["pos_1"][gi, si]] = w[gi, si]
  np.testing.assert_array_equal(r["combine"], want)
  np.testing.assert_array_equal(r["dispatch"], (want != 0).astype(np.float32))
  assert (r["dispatch"].sum(axis=1) <= 1).all()      # one token per slot


def test_v1_switch_dense_equals_index_form():
  rng = np.random.default_rng(34)
  b, l, m, h, e = 2, 48, 16, 24, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = rng.standard_normal((e, m, h)).astype(np.float32) / 4
  wo = rng.standard_normal((e, h, m)).astype(np.float32) / 5
  hp = O.default_hparams(moe_gating="switch", moe_num_experts=e,
                         moe_hidden_size=h, moe_group_size=32,
                         moe_capacity_factor_eval=1.0)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  d, dl, aux = O.moe_layer_v1(x, wg, wi, wo, hp, False, nonpadding=nonpad,
                              dense=True)
  i, il, _ = O.moe_layer_v1(x, wg, wi, wo, hp, False, nonpadding=nonpad,
                            dense=False)
  np.testing.assert_allclose(d, i, rtol=1e-5, atol=1e-5)
  assert dl == il
  assert (d[nonpad == 0] == 0).all()
  assert (d[~aux["kept_1"].reshape(b, l)] == 0).all()
  # a token that kept its slot gets gate * FFN_e(x): check one by hand
  t = int(np.flatnonzero(aux["kept_1"].reshape(-1))[0])
  ex = int(aux["index_1"].reshape(-1)[t])
  xt = x.reshape(-1, m)[t].astype(np.float64)
  ref = np.maximum(xt @ wi[ex].astype(np.float64), 0) @ wo[ex].astype(np.float64)
  np.testing.assert_allclose(d.reshape(-1, m)[t],
                             aux["gate_1"].reshape(-1)[t] * ref, rtol=1e-4,
                             atol=1e-5)
  hp.moe_switch_policy_eval = "sample"
  with pytest.raises(NotImplementedError):
    O.moe_layer_v1(x, wg, wi, wo, hp, False)


# ---- ntlb ("no token left behind") gating ---------------------------------------
def _ntlb_by_token_walk(p64, k, c, imp):
  """transformer/moe.py:903-934 as a walk over (pass, token): pass i offers
  the unrouted tokens, in token order, to their i-th best expert; the expert's
  counter for the pass starts at what it holds and counts every offer, taken
  or not; an offer is taken while the counter stays within the capacity."""
  g, s, e = p64.shape
  order = np.argsort(-p64, axis=-1, kind="stable")[..., :k]
  routed = np.full((g, s), -1)
  slot = np.zeros((g, s), int)
  held = np.zeros((g, e), int)
  for gi in range(g):
    for i in range(k):
      offered = held[gi].copy()
      for si in range(s):
        if routed[gi, si] >= 0 or (imp is not None and imp[gi, si] != 1.0):
          continue
        ex = order[gi, si, i]
        offered[ex] += 1
        if offered[ex] <= c:
          routed[gi, si], slot[gi, si] = i, offered[ex] - 1
          held[gi, ex] += 1
  return order, routed, slot, held


@pytest.mark.parametrize("seed", range(6))
def test_ntlb_against_token_walk_and_float64(seed):
  rng = np.random.default_rng(900 + seed)
  g, s, e = 3, int(rng.integers(30, 80)), int(rng.integers(3, 7))
  k = 1 + seed % 4 if seed % 4 < e else e
  c = s // e + 1
  # expert 0 is everybody's favourite: it overflows in pass 0 while the
  # others keep room for the later passes
  logits = (2 * rng.standard_normal((g, s, e))).astype(np.float32)
  logits[..., 0] += 2.0
  imp = None
  if seed % 2:
    imp = rng.choice(np.array([0.0, 0.5, 1.0, 1.0, 1.0, 1.0, 1.0], np.float32),
                     size=(g, s))
  p64 = scipy.special.softmax(logits.astype(np.float64), axis=-1)
  order, routed, slot, held = _ntlb_by_token_walk(p64, k, c, imp)
  for dense in (False, True):
    r = O.ntlb_gating(logits, c, k, importance=imp, dense=dense)
    np.testing.assert_array_equal(r["topk_index"], order)
    np.testing.assert_array_equal(r["taken_in_pass"], routed)
    np.testing.assert_array_equal(r["kept_1"], routed >= 0)
    np.testing.assert_array_equal(r["fill"], held)
    assert not r["kept_2"].any() and not r["gate_2"].any()
    took = routed >= 0
    ex = np.take_along_axis(order, np.maximum(routed, 0)[..., None], -1)[..., 0]
    np.testing.assert_array_equal(r["index_1"][took], ex[took])
    np.testing.assert_array_equal(r["pos_1"][took], slot[took])
    want = np.take_along_axis(p64, ex[..., None], -1)[..., 0] * took
    np.testing.assert_allclose(r["gate_1"], want, rtol=2e-6)
  # the capacity leaves first choices unserved, so later passes matter
  assert (routed != 0).any()
  if k > 1:
    assert (routed > 0).any()


def test_ntlb_hand_worked_case():
  """4 tokens, 3 experts, capacity 1, k = 2.  First choices 0,0,1,0; second
  choices 1,2,0,1.  Pass 0: token 0 takes expert 0, token 1 overflows it,
  token 2 takes expert 1, token 3 overflows.  Pass 1: token 1 -> expert 2
  (free), token 3 -> expert 1 (full) -> dropped."""
  big, mid, low = 3.0, 1.0, -2.0
  logits = np.array([[[big, mid, low], [big, low, mid], [mid, big, low],
                      [big, mid, low]]], np.float32)
  r = O.ntlb_gating(logits, 1, 2, dense=True)
  p = scipy.special.softmax(logits.astype(np.float64), axis=-1)[0]
  np.testing.assert_array_equal(r["kept_1"][0], [True, True, True, False])
  np.testing.assert_array_equal(r["index_1"][0][:3], [0, 2, 1])
  np.testing.assert_array_equal(r["taken_in_pass"][0], [0, 1, 0, -1])
  np.testing.assert_array_equal(r["pos_1"][0][:3], [0, 0, 0])
  np.testing.assert_allclose(r["gate_1"][0], [p[0, 0], p[1, 2], p[2, 1], 0],
                             rtol=2e-6)
  np.testing.assert_array_equal(r["fill"][0], [1, 1, 1])
  want = np.zeros((4, 3, 1), np.float32)
  want[0, 0, 0], want[1, 2, 0], want[2, 1, 0] = r["gate_1"][0][:3]
  np.testing.assert_array_equal(r["combine"][0], want)


def test_ntlb_with_one_choice_is_switch():
  """k = 1: the one round is _switch_gating's capacity rule (an offer counts
  whether or not it is taken, moe.py:1268-1276 and :908-914) and the loss is
  the same expression."""
  rng = np.random.default_rng(910)
  logits = rng.standard_normal((2, 50, 4)).astype(np.float32)
  imp = rng.choice(np.array([0.0, 1.0], np.float32), size=(2, 50))
  for importance in (None, imp):
    a = O.ntlb_gating(logits, 7, 1, importance=importance, num_microbatches=3)
    b = O.switch_gating(logits, 7, importance=importance, num_microbatches=3)
    for key in ("kept_1", "gate_1", "fill"):
      np.testing.assert_array_equal(a[key], b[key])
    np.testing.assert_array_equal(a["index_1"][a["kept_1"]],
                                  b["index_1"][b["kept_1"]])
    np.testing.assert_array_equal(a["pos_1"][a["kept_1"]],
                                  b["pos_1"][b["kept_1"]])
    np.testing.assert_allclose(a["loss"], b["loss"], rtol=1e-6)


def test_ntlb_loss_closed_forms():
  """loss = E^2 * mean over [G,k,E] of proxy[g,e] * density[g,i,e]
  (moe.py:845-856).  Uniform router: proxy = 1/E, and each pass's density
  sums to 1 over the experts, so the loss is E^2 * (1/E) * 1/E = 1 for any k.
  With importance the product gains the group dim and the mean the factor
  mean(importance == 1)."""
  g, s, e, k = 2, 24, 4, 3
  r = O.ntlb_gating(np.zeros((g, s, e), np.float32), 100, k)
  np.testing.assert_allclose(r["loss"], 1.0, rtol=1e-6)
  # uniform router: every token names experts 0..k-1 in this order
  np.testing.assert_array_equal(r["topk_index"][0, 0], np.arange(k))
  imp = np.ones((g, s), np.float32)
  imp[:, : s // 4] = 0.0
  r2 = O.ntlb_gating(np.zeros((g, s, e), np.float32), 100, k, importance=imp)
  np.testing.assert_allclose(r2["loss"], 0.75, rtol=1e-6)
  rng = np.random.default_rng(911)
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  p = scipy.special.softmax(logits.astype(np.float64), axis=-1)
  order = np.argsort(-p, axis=-1, kind="stable")[..., :k]
  dens = np.stack([(order[..., i, None] == np.arange(e)).mean(axis=1)
                   for i in range(k)], axis=1)               # [G,k,E]
  want = e * e * (p.mean(axis=1)[:, None, :] * dens).mean()
  got = O.ntlb_gating(logits, 5, k, num_microbatches=2)["loss"]
  np.testing.assert_allclose(got, want / 2, rtol=1e-5)


# ---- the bfloat16 softmax of _ntlb_gating (moe.py:825-836) -----------------
def _bf16_rne(v):
  """Round a Python float to 8 significant bits, ties to even, with frexp and
  integer rounding only (shares nothing with the oracle's bit-twiddling
  round_bf16)."""
  import math
  if v == 0.0 or math.isinf(v):
    return v
  mant, exp = math.frexp(v)               # 0.5 <= |mant| < 1
  return math.ldexp(round(mant * 256.0), exp - 8)   # round(): ties to even


def _softmax_bf16_by_hand(row):
  """mtf.softmax (ops.py:5493-5541) on a bfloat16 row, op by op in Python
  floats: every op's result is rounded to bfloat16 (reduce_max and negative
  are exact); the sum is rounded once."""
  import math
  x = [_bf16_rne(float(v)) for v in row]
  m = max(x)
  t = [_bf16_rne(v - m) for v in x]
  u = [_bf16_rne(math.exp(v)) for v in t]
  s = _bf16_rne(sum(u))
  lse = _bf16_rne(_bf16_rne(math.log(s)) + m)
  return [_bf16_rne(math.exp(_bf16_rne(v - lse))) for v in x]


def test_softmax_bf16_hand_worked_rows():
  """Worked with pencil and a table of exp / log:

  [0, 0, 0]: exp(0) = 1 three times, sum 3, log 3 = 1.0986 -> 1.1015625 (ulp
  2^-7: 12.62 -> 13 steps above 1), exp(-1.1015625) = 0.33235 -> 0.33203125
  (ulp 2^-9: 170.16 -> 170).  The float32 chain gives 1/3.

  [1, 0, -1]: t = [0, -1, -2]; exp -> 1, 0.36788 -> 0.3671875 (188.35 -> 188
  steps of 2^-9), 0.13534 -> 0.1357421875 (138.58 -> 139 steps of 2^-10); sum
  1.50293 -> 1.5; log 1.5 = 0.405465 -> 0.40625 (207.6 -> 208 steps of 2^-9);
  lse = 1.40625; exp(-0.40625) = 0.666143 -> 0.66796875 (170.53 -> 171 steps
  of 2^-8), exp(-1.40625) = 0.245060 -> 0.2451171875 (250.94 -> 251 steps of
  2^-10), exp(-2.40625) = 0.090152 -> 0.09033203125 (184.63 -> 185 steps of
  2^-11).  These do not sum to 1: 1.00341796875."""
  p = O.softmax_bf16(np.array([[0, 0, 0], [1, 0, -1]], np.float32))
  np.testing.assert_array_equal(p[0], [0.33203125] * 3)
  np.testing.assert_array_equal(p[1], [0.66796875, 0.2451171875, 0.09033203125])
  assert p.dtype == np.float32


@pytest.mark.parametrize("seed", range(4))
def test_softmax_bf16_against_python_float_chain(seed):
  rng = np.random.default_rng(930 + seed)
  e = int(rng.integers(2, 9))
  logits = (3 * rng.standard_normal((40, e))).astype(np.float32)
  got = O.softmax_bf16(logits)
  want = np.array([_softmax_bf16_by_hand(r) for r in logits], np.float64)
  np.testing.assert_array_equal(got.astype(np.float64), want)


def test_softmax_bf16_properties():
  rng = np.random.default_rng(934)
  logits = (2 * rng.standard_normal((3, 50, 16))).astype(np.float32)
  p = O.softmax_bf16(logits)
  # every value is a bfloat16
  assert not (p.view(np.uint32) & 0xFFFF).any()
  # the logits are rounded first: feeding the rounded logits changes nothing
  np.testing.assert_array_equal(p, O.softmax_bf16(O.round_bf16(logits)))
  # close to the exact softmax of the rounded logits: seven roundings of
  # 2^-9 relative each, three of them on exponents of size <= ~8
  exact = scipy.special.softmax(O.round_bf16(logits).astype(np.float64), -1)
  np.testing.assert_allclose(p, exact, rtol=0.08)
  # where every op's result is a bfloat16 anyway the two chains agree bit for
  # bit: one-hot rows (exp(-200) = 0, sum 1, log 0) ...
  onehot = np.full((5, 6), -200.0, np.float32)
  onehot[np.arange(5), [0, 3, 5, 1, 2]] = 0.0
  np.testing.assert_array_equal(O.softmax_bf16(onehot), O.softmax(onehot))
  np.testing.assert_array_equal(O.softmax(onehot).sum(-1), np.ones(5))
  # ... and the dispatcher: only ntlb with bfloat16 activations uses it
  for gating in ("top_2", "switch", "switch_max", "expert_selection", "ntlb"):
    for act in ("float32", "bfloat16"):
      want = O.softmax_bf16 if (gating, act) == ("ntlb", "bfloat16") else O.softmax
      np.testing.assert_array_equal(O.router_softmax(logits, gating, act),
                                    want(logits))


def test_ntlb_bfloat16_ties_go_to_the_lower_index():
  """bfloat16 probabilities tie often.  Row [0, 0, 0, -1]: three experts at
  the same probability, named in index order (repeated first-arg-max,
  ops.py:5009-5014); capacity 1 and k = 3 then place tokens 0, 1, 2 on experts
  0, 1, 2 in passes 0, 1, 2 and leave token 3 out."""
  logits = np.tile(np.array([0, 0, 0, -1], np.float32), (1, 4, 1))
  # bfloat16 chain by hand: exp(0) = 1 x3, exp(-1) -> 0.3671875, sum 3.3671875
  # -> 3.375 (ulp 2^-6), log = 1.21640 -> 1.21875 (ulp 2^-7: 27.7 -> 28),
  # exp(-1.21875) = 0.29560 -> 0.294921875 (ulp 2^-9: 151.3 -> 151)
  r = O.ntlb_gating(logits, 1, 3, act_dtype="bfloat16")
  np.testing.assert_array_equal(r["topk_index"][0], [[0, 1, 2]] * 4)
  np.testing.assert_array_equal(r["kept_1"][0], [True, True, True, False])
  np.testing.assert_array_equal(r["index_1"][0][:3], [0, 1, 2])
  np.testing.assert_array_equal(r["taken_in_pass"][0], [0, 1, 2, -1])
  np.testing.assert_array_equal(r["gate_1"][0], [0.294921875] * 3 + [0.0])
  # float32 activations: the same routing with the float32 probability
  r32 = O.ntlb_gating(logits, 1, 3)
  np.testing.assert_array_equal(r32["index_1"], r["index_1"])
  np.testing.assert_allclose(r32["gate_1"][0][:3], 1 / (3 + np.exp(-1.0)),
                             rtol=1e-6)


def test_ntlb_bfloat16_rounds_the_logits_first():
  """Two logits that differ in float32 but round to the same bfloat16 tie in
  the reference (its projection's result is a bfloat16 tensor): the lower
  index comes first, whichever is larger in float32."""
  logits = np.array([[[1.0, 1.001, -3.0]]], np.float32)
  assert O.ntlb_gating(logits, 4, 2)["topk_index"][0, 0].tolist() == [1, 0]
  got = O.ntlb_gating(logits, 4, 2, act_dtype="bfloat16")
  assert got["topk_index"][0, 0].tolist() == [0, 1]


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_ntlb_dense_tensors_match_index_record(act_dtype):
  rng = np.random.default_rng(912)
  g, s, e, c, k = 2, 40, 5, 5, 3
  logits = (2 * rng.standard_normal((g, s, e))).astype(np.float32)
  r = O.ntlb_gating(logits, c, k, act_dtype=act_dtype, dense=True)
  want = np.zeros((g, s, e, c), np.float32)
  w = O.cast_act(r["gate_1"], act_dtype)
  for gi in range(g):
    for si in range(s):
      if r["kept_1"][gi, si]:
        want[gi, si, r["index_1"][gi, si], r["pos_1"][gi, si]] = w[gi, si]
  np.testing.assert_array_equal(r["combine"], want)
  np.testing.assert_array_equal(r["dispatch"], (want != 0).astype(np.float32))
  assert (r["dispatch"].sum(axis=1) <= 1).all()      # one token per slot
  assert (r["taken_in_pass"] > 0).any()


def test_v1_ntlb_dense_equals_index_form():
  rng = np.random.default_rng(913)
  b, l, m, h, e = 2, 48, 16, 24, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = rng.standard_normal((e, m, h)).astype(np.float32) / 4
  wo = rng.standard_normal((e, h, m)).astype(np.float32) / 5
  hp = O.default_hparams(moe_gating="ntlb", moe_num_experts=e,
                         moe_hidden_size=h, moe_group_size=32,
                         moe_capacity_factor_eval=1.0, moe_ntlb_top_k=2)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  d, dl, aux = O.moe_layer_v1(x, wg, wi, wo, hp, False, nonpadding=nonpad,
                              dense=True)
  i, il, _ = O.moe_layer_v1(x, wg, wi, wo, hp, False, nonpadding=nonpad,
                            dense=False)
  np.testing.assert_allclose(d, i, rtol=1e-5, atol=1e-5)
  assert dl == il
  assert (d[nonpad == 0] == 0).all()
  t = int(np.flatnonzero(aux["taken_in_pass"].reshape(-1) == 1)[0])   # a second choice
  ex = int(aux["index_1"].reshape(-1)[t])
  xt = x.reshape(-1, m)[t].astype(np.float64)
  ref = np.maximum(xt @ wi[ex].astype(np.float64), 0) @ wo[ex].astype(np.float64)
  np.testing.assert_allclose(d.reshape(-1, m)[t],
                             aux["gate_1"].reshape(-1)[t] * ref, rtol=1e-4,
                             atol=1e-5)


# ---- switch_max gating ----------------------------------------------------------
def test_top_k_matches_iterative_top_1():
  """mtf.top_k lowers 1 < k < 5 as repeated top_1 with the taken entries pushed
  down by 1e9 (ops.py:4988-5017) and other k as tf.math.top_k (lower index first
  on ties): both select what the stable descending sort selects."""
  rng = np.random.default_rng(51)
  x = np.round(rng.random((3, 40, 5)) * 6) / 6        # many exact ties
  x = x.astype(np.float32)
  for k in (1, 2, 4, 7):
    vals, idx = O.top_k_lowest_index_first(x, k, axis=1)      # over the 40
    y = x.copy()
    for i in range(k):
      m = y.max(axis=1)
      am = y.argmax(axis=1)                                    # first max
      np.testing.assert_array_equal(idx[..., i], am)
      np.testing.assert_array_equal(vals[..., i], np.take_along_axis(x, am[:, None, :], 1)[:, 0, :])
      np.put_along_axis(y, am[:, None, :], -1e9, axis=1)
      del m


@pytest.mark.parametrize("seed", range(4))
def test_switch_max_brute_force(seed):
  """Per (group, expert): the tokens that chose the expert, sorted by gate
  descending (token order on ties), fill slots 0..C-1; the rest are dropped."""
  rng = np.random.default_rng(400 + seed)
  g, s, e = 2, int(rng.integers(6, 80)), int(rng.integers(2, 7))
  c = int(rng.integers(1, s // e + 3))
  scale = 0.0 if seed == 3 else 1.0                    # seed 3: all gates tie
  logits = (rng.standard_normal((g, s, e)) * scale).astype(np.float32)
  imp = None
  if seed % 2:
    imp = rng.choice(np.array([0.0, 0.5, 1.0], np.float32), size=(g, s))
  p = O.softmax(logits)
  for dense in (False, True):
    r = O.switch_max_gating(logits, c, importance=imp, dense=dense)
    np.testing.assert_array_equal(r["index_1"], p.argmax(-1))
    for gi in range(g):
      for ex in range(e):
        chose = [t for t in range(s) if r["index_1"][gi, t] == ex and
                 (imp is None or imp[gi, t] == 1.0)]
        chose.sort(key=lambda t: (-p[gi, t, ex], t))
        for rank, t in enumerate(chose):
          assert r["kept_1"][gi, t] == (rank < c)
          if rank < c:
            assert r["pos_1"][gi, t] == rank
            assert r["gate_1"][gi, t] == p[gi, t, ex]
          else:
            assert r["gate_1"][gi, t] == 0
        assert r["fill"][gi, ex] == min(len(chose), c)
    if imp is not None:
      assert not r["kept_1"][imp != 1.0].any()
    if dense:
      want = np.zeros((g, s, e, c), np.float32)
      kk = r["kept_1"]
      for gi, t in zip(*np.nonzero(kk)):
        want[gi, t, r["index_1"][gi, t], r["pos_1"][gi, t]] = r["gate_1"][gi, t]
      np.testing.assert_array_equal(r["combine"], want)
      np.testing.assert_array_equal(r["dispatch"], (want != 0).astype(np.float32))


def test_switch_max_equals_switch_without_overflow():
  """With room for every token the two routers keep the same tokens with the
  same gates and the same loss; only the slot order differs."""
  rng = np.random.default_rng(52)
  logits = rng.standard_normal((2, 50, 4)).astype(np.float32)
  a = O.switch_gating(logits, 50)
  b = O.switch_max_gating(logits, 50)
  for k in ("index_1", "kept_1", "fill"):
    np.testing.assert_array_equal(a[k], b[k])
  np.testing.assert_array_equal(a["gate_1"], b["gate_1"])
  assert a["loss"] == b["loss"]
  # under overflow switch_max keeps the confident tokens, switch the early ones
  c = 5
  a, b = O.switch_gating(logits, c), O.switch_max_gating(logits, c)
  np.testing.assert_array_equal(a["fill"], b["fill"])
  assert b["gate_1"].sum() > a["gate_1"].sum()


# ---- expert_selection gating ------------------------------------------------------
@pytest.mark.parametrize("seed", range(3))
def test_expert_selection_brute_force(seed):
  """Per (group, expert): softmax over the group's tokens in float64, tokens
  sorted by probability descending (token order on ties), the first C fill the
  slots; a token's weights are its probabilities over the number of experts
  that chose it (transformer/moe.py:1099-1123)."""
  rng = np.random.default_rng(500 + seed)
  g, s, e = 2, int(rng.integers(8, 60)), int(rng.integers(2, 6))
  c = int(rng.integers(1, s // 2))
  quantum = 0.5 if seed == 2 else 0.0                   # seed 2: exact ties
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  if quantum:
    logits = (np.round(logits / quantum) * quantum).astype(np.float32)
  imp = rng.choice(np.array([0.0, 1.0], np.float32), size=(g, s), p=[0.2, 0.8])
  masked = logits.astype(np.float64) + (imp == 0)[..., None] * -1e9
  p64 = scipy.special.softmax(masked, axis=1)
  for dense in (False, True):
    r = O.expert_selection_gating(logits, c, imp, dense=dense)
    count = np.zeros((g, s), int)
    for gi in range(g):
      for ex in range(e):
        order = sorted(range(s), key=lambda t: (-O.F32(p64[gi, t, ex]), t))
        if not quantum:
          np.testing.assert_array_equal(r["slot_token"][gi, ex], order[:c])
        count[gi][r["slot_token"][gi, ex]] += 1
    for gi in range(g):
      for ex in range(e):
        tok = r["slot_token"][gi, ex]
        np.testing.assert_allclose(
            r["slot_weight"][gi, ex], p64[gi, tok, ex] / count[gi, tok],
            rtol=3e-6, atol=1e-30)
        # probabilities descend along the slots, ties in token order
        pv = p64[gi, tok, ex]
        assert (np.diff(pv) <= 1e-12).all()
        if quantum:
          same = np.isclose(np.diff(pv), 0, atol=1e-15)
          assert (np.diff(tok)[same] > 0).all()
    if dense:
      want = np.zeros((g, s, e, c), np.float32)
      disp = np.zeros((g, s, e, c), np.float32)
      for gi in range(g):
        for ex in range(e):
          want[gi, r["slot_token"][gi, ex], ex, np.arange(c)] = \
              r["slot_weight"][gi, ex]
          disp[gi, r["slot_token"][gi, ex], ex, np.arange(c)] = 1.0
      np.testing.assert_allclose(r["combine"], want, rtol=1e-6)
      # the dispatch tensor is the one-hot itself, whatever the weight
      np.testing.assert_array_equal(r["dispatch"], disp)
      assert (r["dispatch"].sum(axis=1) == 1).all()     # every slot is filled


def test_expert_selection_loss_closed_forms():
  """loss = mean_{g,s}(agg^2 * sum_s importance) * S with agg = mean_e p
  (moe.py:1125-1147).  Uniform logits: p = 1/n over the n unmasked tokens,
  loss = 1 whatever the mask; all mass on one token: loss = S."""
  s, e = 32, 4
  ones = np.ones((2, s), np.float32)
  np.testing.assert_allclose(
      O.expert_selection_gating(np.zeros((2, s, e), np.float32), 4, ones)["loss"],
      1.0, rtol=1e-5)
  imp = ones.copy()
  imp[:, ::2] = 0.0
  np.testing.assert_allclose(
      O.expert_selection_gating(np.zeros((2, s, e), np.float32), 4, imp)["loss"],
      1.0, rtol=1e-5)
  peak = np.zeros((1, s, e), np.float32)
  peak[0, 5] = 60.0
  np.testing.assert_allclose(
      O.expert_selection_gating(peak, 4, ones[:1])["loss"], s, rtol=1e-5)
  np.testing.assert_allclose(
      O.expert_selection_gating(peak, 4, ones[:1], num_microbatches=4)["loss"],
      s / 4, rtol=1e-5)


def test_v1_expert_selection_dense_equals_index_form():
  rng = np.random.default_rng(53)
  b, l, m, h, e = 2, 48, 16, 24, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = rng.standard_normal((e, m, h)).astype(np.float32) / 4
  wo = rng.standard_normal((e, h, m)).astype(np.float32) / 5
  hp = O.default_hparams(moe_gating="expert_selection", moe_num_experts=e,
                         moe_hidden_size=h, moe_group_size=32,
                         moe_capacity_factor_eval=2.0,
                         moe_switch_policy_eval="argmax")
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  d, dl, aux = O.moe_layer_v1(x, wg, wi, wo, hp, False, nonpadding=nonpad,
                              dense=True)
  i, il, _ = O.moe_layer_v1(x, wg, wi, wo, hp, False, nonpadding=nonpad,
                            dense=False)
  np.testing.assert_allclose(d, i, rtol=1e-5, atol=1e-6)
  assert dl == il and aux["capacity"] == 16
  # tokens nobody chose output zero; a chosen one is the weighted FFN sum
  chosen = np.zeros((aux["num_groups"], aux["group_size"]), bool)
  for gi in range(aux["num_groups"]):
    chosen[gi][aux["slot_token"][gi].reshape(-1)] = True
  assert (d.reshape(chosen.shape + (m,))[~chosen] == 0).all() and chosen.any()
  with pytest.raises(ValueError):
    O.moe_layer_v1(x, wg, wi, wo, hp, False)


# ---- the layers ----------------------------------------------------------------
def _hp(**kw):
  base = dict(moe_second_policy_train="all", moe_second_policy_eval="all")
  base.update(kw)
  return O.default_hparams(**base)


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_v1_dense_equals_index_form(act_dtype):
  rng = np.random.default_rng(12)
  b, l, m, h, e = 2, 48, 16, 24, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = rng.standard_normal((e, m, h)).astype(np.float32) / 4
  wo = rng.standard_normal((e, h, m)).astype(np.float32) / 5
  hp = _hp(moe_num_experts=e, moe_hidden_size=h, moe_group_size=32,
           moe_capacity_factor_train=1.0)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  d, dl, aux = O.moe_layer_v1(x, wg, wi, wo, hp, True, act_dtype,
                              nonpadding=nonpad, dense=True)
  i, il, _ = O.moe_layer_v1(x, wg, wi, wo, hp, True, act_dtype,
                            nonpadding=nonpad, dense=False)
  tol = 1e-2 if act_dtype == "bfloat16" else 1e-5
  np.testing.assert_allclose(d, i, rtol=tol, atol=tol)
  assert dl == il and aux["num_groups"] == 3 and aux["group_size"] == 32
  assert (d[nonpad == 0] == 0).all()
  # a token that lost both choices outputs exactly zero
  lost = ~(aux["kept_1"] | aux["kept_2"]).reshape(b, l)
  assert (d[lost] == 0).all()


def test_v1_single_expert_is_a_dense_ffn():
  """E = 2 identical experts, capacity for everything: gates sum to 1, so the
  layer equals one feed-forward network applied to every token."""
  rng = np.random.default_rng(13)
  b, l, m, h = 1, 16, 8, 12
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wi1 = rng.standard_normal((m, h)).astype(np.float32)
  wo1 = rng.standard_normal((h, m)).astype(np.float32)
  hp = _hp(moe_num_experts=2, moe_hidden_size=h, moe_group_size=16,
           moe_capacity_factor_train=4.0)
  out, _, _ = O.moe_layer_v1(x, rng.standard_normal((m, 2)).astype(np.float32),
                             np.stack([wi1, wi1]), np.stack([wo1, wo1]), hp, True)
  want = np.maximum(x.astype(np.float64) @ wi1, 0) @ wo1
  np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-4)


def test_v2_with_one_outer_expert_reduces_to_v1():
  """x = 1 outer group with capacity for every token: the outer level passes
  every token through with gate 1/(1+1e-9) rounding to 1, importance 1, and the
  inner level is a v1 layer over the same tokens in the same order."""
  rng = np.random.default_rng(14)
  b, l, m, h, ye = 2, 32, 8, 16, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  w_outer = rng.standard_normal((m, 1)).astype(np.float32)
  w_inner = rng.standard_normal((1, m, ye)).astype(np.float32)
  wi = rng.standard_normal((ye, 1, m, h)).astype(np.float32) / 3
  wo = rng.standard_normal((ye, 1, h, m)).astype(np.float32) / 4
  hp2 = _hp(moe_num_experts=[1, ye], moe_hidden_size=h, moe_group_size=32,
            moe_capacity_factor_train=1.0, moe_capacity_factor_second_level=1.5,
            moe_min_expert_capacity=1)
  out2, loss2, aux = O.moe_layer_v2(x, w_outer, w_inner, wi, wo, hp2, True)
  assert aux["capacity_x"] == 32 and aux["groups_y"] == (2, 32)
  assert aux["outer"]["kept_1"].all()
  hp1 = _hp(moe_num_experts=ye, moe_hidden_size=h, moe_group_size=32,
            moe_capacity_factor_train=1.5, moe_min_expert_capacity=1)
  out1, loss1, _ = O.moe_layer_v1(x, w_inner[0], wi[:, 0], wo[:, 0], hp1, True)
  np.testing.assert_allclose(out2, out1, rtol=1e-5, atol=1e-6)
  # outer loss with one expert: density = proxy = 1 -> 1; total = (1 + inner)
  np.testing.assert_allclose(loss2, (1.0 + loss1 / 1e-2) * 1e-2, rtol=1e-5)


def test_v2_importance_mapping():
  """importance = 0.5 * ((w > 0.5) + (w > 0)) on the slot weights
  (transformer/moe.py:725-727)."""
  w = np.array([0.0, 0.3, 0.5, 0.7], np.float32)
  imp = np.float32(0.5) * ((w > 0.5).astype(np.float32) + (w > 0).astype(np.float32))
  np.testing.assert_array_equal(imp, [0.0, 0.5, 0.5, 1.0])
  rng = np.random.default_rng(15)
  x = rng.standard_normal((2, 64, 8)).astype(np.float32)
  hp = _hp(moe_num_experts=[4, 4], moe_hidden_size=8, moe_group_size=32)
  _, _, aux = O.moe_layer_v2(
      x, rng.standard_normal((8, 4)).astype(np.float32),
      rng.standard_normal((4, 8, 4)).astype(np.float32),
      rng.standard_normal((4, 4, 8, 8)).astype(np.float32),
      rng.standard_normal((4, 4, 8, 8)).astype(np.float32), hp, True)
  imp = aux["importance_inner"]
  assert set(np.unique(imp)) <= {0.0, 0.5, 1.0}
  n_first = int(aux["outer"]["kept_1"].sum())
  # every kept first choice has gate > 0.5 here (no exact ties), so it becomes 1.0
  assert int((imp == 1.0).sum()) == n_first
  assert int((imp == 0.5).sum()) == int(aux["outer"]["kept_2"].sum())


def test_golden_fixture():
  """Small committed input/output vectors of the oracle itself (guards the
  oracle against accidental edits; generated by tests/golden/make_golden.py)."""
  path = os.path.join(GOLDEN, "top2_gating_small.json")
  with open(path) as f:
    gold = json.load(f)
  logits = np.array(gold["logits"], np.float32)
  r = O.top_2_gating(logits, gold["capacity"])
  for k in ("index_1", "index_2", "pos_1", "pos_2"):
    np.testing.assert_array_equal(r[k], np.array(gold[k]))
  np.testing.assert_array_equal(r["kept_1"], np.array(gold["kept_1"], bool))
  np.testing.assert_array_equal(r["kept_2"], np.array(gold["kept_2"], bool))
  np.testing.assert_allclose(r["gate_1"], np.array(gold["gate_1"]), rtol=1e-6)
  np.testing.assert_allclose(r["loss"], gold["loss"], rtol=1e-6)


def test_switch_golden_fixture():
  path = os.path.join(GOLDEN, "switch_gating_small.json")
  with open(path) as f:
    gold = json.load(f)
  r = O.switch_gating(np.array(gold["logits"], np.float32), gold["capacity"],
                      importance=np.array(gold["importance"], np.float32),
                      train=True, z_loss=gold["z_loss"],
                      num_microbatches=gold["num_microbatches"])
  for k in ("index_1", "pos_1"):
    np.testing.assert_array_equal(r[k], np.array(gold[k]))
  np.testing.assert_array_equal(r["kept_1"], np.array(gold["kept_1"], bool))
  np.testing.assert_allclose(r["gate_1"], np.array(gold["gate_1"]), rtol=1e-6)
  np.testing.assert_allclose(r["loss"], gold["loss"], rtol=1e-6)


def test_gated_expert_hidden_against_float64():
  """Product of dense layers (gated units): an independent float64 evaluation,
  the one-factor list equals the plain layer, and a zero kernel in one linear
  factor zeroes the output."""
  rng = np.random.default_rng(77)
  e, r, m, h, n = 3, 10, 6, 8, 5
  xe = rng.standard_normal((e, r, m)).astype(np.float32)
  wi0 = rng.standard_normal((e, m, h)).astype(np.float32)
  wi1 = rng.standard_normal((e, m, h)).astype(np.float32)
  wo = rng.standard_normal((e, h, n)).astype(np.float32)
  x64, a64, b64, o64 = (v.astype(np.float64) for v in (xe, wi0, wi1, wo))
  for acts, f0, f1 in (
      (["gelu", "linear"], None, lambda v: v),
      (["linear", "sigmoid"], lambda v: v, scipy.special.expit),
      (["relu", "swish"], lambda v: np.maximum(v, 0),
       lambda v: v * scipy.special.expit(v)),
      (["tanh", "relu"], np.tanh, lambda v: np.maximum(v, 0))):
    if f0 is None:      # tanh-approximated gelu, ops.py gelu
      f0 = lambda v: 0.5 * v * (1 + np.tanh(
          np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3)))
    want = (f0(x64 @ a64) * f1(x64 @ b64)) @ o64
    got = O.expert_ffn(xe, [wi0, wi1], wo, acts, "float32")
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
    # the factors commute
    swapped = O.expert_ffn(xe, [wi1, wi0], wo, acts[::-1], "float32")
    np.testing.assert_allclose(swapped, got, rtol=1e-5, atol=1e-5)
  np.testing.assert_array_equal(
      O.expert_ffn(xe, [wi0], wo, ["relu"], "bfloat16"),
      O.expert_ffn(xe, wi0, wo, "relu", "bfloat16"))
  np.testing.assert_array_equal(
      O.expert_ffn(xe, [wi0, np.zeros_like(wi1)], wo, ["relu", "linear"],
                   "float32"), np.zeros((e, r, n), np.float32))
  with pytest.raises(ValueError):
    O.expert_ffn(xe, [wi0, wi1], wo, ["relu"], "float32")


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_hidden_dropout_noise(act_dtype):
  """The dropout multiplier: zero or 1 / keep_prob in the tensor's dtype, strict
  comparison, scalars rounded to that dtype (checked against torch's own
  arithmetic in that dtype)."""
  import torch
  tdt = torch.float32 if act_dtype == "float32" else torch.bfloat16
  rng = np.random.default_rng(5)
  for keep in (0.5, 0.9, 0.75, 0.3):
    u = O.cast_act(rng.random((4, 50, 7)).astype(np.float32), act_dtype)
    keep_t = torch.tensor(keep, dtype=tdt)
    u[0, 0, 0] = float(keep_t)                          # not strictly below
    u[0, 0, 1] = 0.0
    noise = O.hidden_dropout_noise(u, keep, act_dtype)
    want = ((torch.from_numpy(u).to(tdt) < keep_t).to(tdt) / keep_t).float().numpy()
    np.testing.assert_array_equal(noise, want)
    assert noise[0, 0, 0] == 0 and noise[0, 0, 1] > 1
    assert set(np.unique(noise)) == {0.0, float(torch.tensor(1.0, dtype=tdt) / keep_t)}
    assert abs(noise.mean() - 1.0) < 0.15
  # the layer: dropped hidden units change the output, evaluation ignores it,
  # and keep_prob -> noise of all ones is the plain layer
  e, m, hdim, group = 4, 8, 12, 32
  x = rng.standard_normal((2, 32, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = rng.standard_normal((e, m, hdim)).astype(np.float32)
  wo = rng.standard_normal((e, hdim, m)).astype(np.float32)
  hp = _hp(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
           moe_dropout_rate=0.5)
  hp0 = _hp(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group)
  cap = O.expert_capacity(group, hp.moe_capacity_factor_train, e,
                          hp.moe_min_expert_capacity)
  hu = rng.random((e, 2 * cap, hdim)).astype(np.float32)
  plain, _, _ = O.moe_layer_v1(x, wg, wi, wo, hp0, True, act_dtype, dense=False)
  with pytest.raises(NotImplementedError):
    O.moe_layer_v1(x, wg, wi, wo, hp, True, act_dtype, dense=False)
  dropped, _, _ = O.moe_layer_v1(x, wg, wi, wo, hp, True, act_dtype,
                                 dense=False, hidden_uniform=hu)
  assert np.abs(dropped - plain).max() > 0.1
  ev, _, _ = O.moe_layer_v1(x, wg, wi, wo, hp, False, act_dtype, dense=False)
  ev0, _, _ = O.moe_layer_v1(x, wg, wi, wo, hp0, False, act_dtype, dense=False)
  np.testing.assert_array_equal(ev, ev0)
  # all units kept with keep_prob 0.5: exactly twice the plain hidden tensor,
  # hence (a power of two) exactly twice the plain output
  twice, _, _ = O.moe_layer_v1(x, wg, wi, wo, hp, True, act_dtype, dense=False,
                               hidden_uniform=np.zeros_like(hu))
  np.testing.assert_allclose(twice, 2 * plain, rtol=1e-2 if act_dtype ==
                             "bfloat16" else 1e-5, atol=1e-5)


# ---- backward -------------------------------------------------------------------
_F64_ACT = {
    "relu": lambda v: np.maximum(v, 0.0),
    "linear": lambda v: v,
    "gelu": lambda v: 0.5 * v * (1 + np.tanh(
        np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3))),
    "sigmoid": scipy.special.expit,
    "tanh": np.tanh,
    "swish": lambda v: v * scipy.special.expit(v),
}


def _f64_layer(x, wg, wi, wo, aux, gating, m1, coef, mb, z_loss, mult=None,
               hidden_noise=None, density_2=None, activation="relu"):
  """Independent float64 forward of the v1 layer with the ROUTING HELD FIXED
  (experts, kept masks and density counts taken from `aux`): a smooth function
  of (x, wg, wi, wo) whose central differences pin the oracle's backward."""
  g, s, _ = x.shape
  e = wg.shape[1]
  logits = (x if mult is None else x * mult) @ wg     # the router's own input
  if gating == "expert_selection":
    # every expert holds `capacity` slots; softmax over the group's tokens per
    # expert; chosen[g,s,e] and the number of experts per token held fixed
    imp = aux["_importance"].astype(np.float64)
    pc = scipy.special.softmax(logits + (imp == 0)[..., None] * -1e9, axis=1)
    chosen = np.zeros((g, s, e))
    for gi in range(g):
      for ei in range(e):
        chosen[gi, aux["slot_token"][gi, ei], ei] = 1.0
    recip = 1.0 / np.maximum(chosen.sum(-1), 1.0)
    out = 0.0
    for ei in range(e):
      h = 1.0
      for w_f, a_f in zip(wi if isinstance(wi, list) else [wi],
                          activation if isinstance(activation, list)
                          else [activation]):
        h = h * _F64_ACT[a_f](x @ w_f[ei])
      out = out + (chosen[..., ei] * pc[..., ei] * recip)[..., None] * (h @ wo[ei])
    agg = pc.mean(-1) * (imp == 1)
    aux_loss = (agg ** 2 * imp.sum(-1, keepdims=True)).mean() * s / mb
    return out, aux_loss * coef
  p = scipy.special.softmax(logits, axis=-1)
  rows = np.arange(g)[:, None], np.arange(s)[None, :]
  i1, i2 = aux["index_1"], aux["index_2"]
  k1, k2 = aux["kept_1"].astype(np.float64), aux["kept_2"].astype(np.float64)

  wis = wi if isinstance(wi, list) else [wi]
  acts = activation if isinstance(activation, list) else [activation]

  def ffn(idx, pos=None):
    h = 1.0
    for w_f, a_f in zip(wis, acts):      # a product of dense layers
      h = h * _F64_ACT[a_f](np.einsum("gsm,gsmh->gsh", x, w_f[idx]))
    if hidden_noise is not None:          # [E, G, C, H], per expert slot
      cap = hidden_noise.shape[2]
      h = h * hidden_noise[idx, np.arange(g)[:, None], np.minimum(pos, cap - 1)]
    return np.einsum("gsh,gshn->gsn", h, wo[idx])
  onehot1 = (i1[..., None] == np.arange(e)).astype(np.float64)
  if gating == "top_2":
    g1 = p[rows + (i1,)] * m1
    g2 = p[rows + (i2,)] * (1.0 - (i2 == i1) * m1)
    den = g1 + g2 + 1e-9
    out = ((g1 / den * k1)[..., None] * ffn(i1, aux["pos_1"])
           + (g2 / den * k2)[..., None] * ffn(i2, aux["pos_2"]))
    density = (onehot1 * m1[..., None]).mean(1)
    proxy = (p * m1[..., None]).mean(1)
    aux_loss = (proxy * density).mean() * e * e
    if density_2 is not None:     # the second-place term, its density held fixed
      q = p * (1.0 - onehot1 * m1[..., None])
      proxy_2 = (q / (q.sum(-1, keepdims=True) + 1e-9)).mean(1)
      aux_loss = aux_loss + 0.5 * (proxy_2 * density_2).mean() * e * e
    aux_loss = aux_loss / mb
  elif gating == "ntlb":
    out = (p[rows + (i1,)] * m1 * k1)[..., None] * ffn(i1, aux["pos_1"])
    topk = aux["topk_index"]                                  # [G,S,k] fixed
    density = (topk[..., None] == np.arange(e)).mean(1)       # [G,k,E]
    proxy = p.mean(1)                                         # [G,E]
    aux_loss = (proxy[:, None, :, None] * m1[:, None, None, :]
                * density[..., None]).mean() * e * e / mb
  else:
    out = (p[rows + (i1,)] * m1 * k1)[..., None] * ffn(i1, aux["pos_1"])
    density = onehot1.mean(1)
    proxy = p.mean(1)
    aux_loss = (proxy[:, :, None] * m1[:, None, :] * density[:, :, None]
                ).mean() * e * e / mb
    if z_loss is not None:
      lse = scipy.special.logsumexp(logits, axis=-1)
      aux_loss = aux_loss + z_loss * (lse ** 2 * m1).sum() / (m1.sum() * mb)
  return out, aux_loss * coef


@pytest.mark.parametrize("gating", ["top_2", "switch", "switch_max", "ntlb",
                                    "switch+jitter", "switch+dropout",
                                    "ntlb+jitter", "switch+sample",
                                    "top_2+hidden", "top_2+loss2",
                                    "top_2+act:gelu", "switch+act:swish",
                                    "top_2+act:gelu*linear",
                                    "switch+act:tanh*sigmoid*relu",
                                    "expert_selection",
                                    "expert_selection+jitter"])
def test_backward_against_central_differences(gating):
  gating, _, perturb = gating.partition("+")
  hidden = perturb == "hidden"      # dropout on the experts' hidden tensor
  loss2 = perturb == "loss2"        # moe_use_second_place_loss
  activation = "relu"
  if perturb.startswith("act:"):    # other expert activations, gated units
    activation = perturb[4:].split("*")
    activation = activation if len(activation) > 1 else activation[0]
    hidden = len(activation) == 3 and isinstance(activation, list)
    perturb = ""
  if hidden or loss2:
    perturb = ""
  rng = np.random.default_rng(61)
  b, l, m, h, e, group = 2, 24, 6, 10, 4, 24
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = (rng.standard_normal((e, m, h)) / 2).astype(np.float32)
  if isinstance(activation, list):
    wi = [wi] + [(rng.standard_normal((e, m, h)) / 2).astype(np.float32)
                 for _ in activation[1:]]
  wo = (rng.standard_normal((e, h, m)) / 3).astype(np.float32)
  nonpad = (rng.random((b, l)) < 0.8).astype(np.float32)
  d_out = rng.standard_normal((b, l, m)).astype(np.float32)
  d_loss, mb = 1.7, 2
  hp = _hp(moe_gating=gating, moe_num_experts=e, moe_hidden_size=h,
           moe_group_size=group, moe_capacity_factor_train=1.2,
           moe_min_expert_capacity=2, moe_loss_coef=0.5,
           moe_switch_policy_train=("sample" if perturb == "sample" else
                                    "input_" + perturb) if perturb else "argmax",
           moe_switch_temperature=2.0,
           moe_switch_jitter=0.3, moe_switch_dropout=0.25, moe_ntlb_top_k=3,
           moe_z_loss=0.3 if gating == "switch" else None,
           moe_dropout_rate=0.4 if hidden else 0.0,
           moe_use_second_place_loss=loss2,
           moe_second_policy_train="threshold" if loss2 else "all",
           moe_second_threshold_train=0.3)
  noise = rng.random((b, l, m)).astype(np.float32) if perturb else None
  su = rng.random((b * l // group, group, e)).astype(np.float32)
  hu = hnoise = None
  if hidden:
    groups = b * l // group
    cap = O.expert_capacity(group, 1.2, e, 2)
    hu = rng.random((e, groups * cap, h)).astype(np.float32)
    hnoise = ((hu < np.float32(0.6)) / np.float32(0.6)).astype(
        np.float64).reshape(e, groups, cap, h)
    assert 0.3 < (hnoise == 0).mean() < 0.5
  got = O.moe_layer_v1_backward(x, wg, wi, wo, hp, True, "float32", d_out,
                                d_loss, nonpadding=nonpad, num_microbatches=mb,
                                gate_noise=noise, sample_uniform=su,
                                hidden_uniform=hu, activation=activation)
  aux = got["aux"]
  mult = None
  if gating == "expert_selection":
    aux = dict(aux, _importance=nonpad.reshape(b, l))
    counts = np.zeros((b, l))
    for gi in range(b):
      for ei in range(e):
        counts[gi, aux["slot_token"][gi, ei]] += 1
    assert (counts == 0).any() and (counts > 1).any()    # none / several experts
    if perturb:
      mult = aux["gate_mult"].astype(np.float64).reshape(b, l, m)
    m1 = z = None
    def scalar(xv, wgv, wiv, wov):
      out, loss = _f64_layer(xv.reshape(b, l, m), wgv, wiv, wov, aux, gating,
                             None, 0.5, mb, None, mult)
      return (out * d_out.reshape(out.shape)).sum() + d_loss * loss
    base = [a.astype(np.float64) for a in (x.reshape(b, l, m), wg, wi, wo)]
    grads = [got["dx"].reshape(b, l, m), got["dw_gate"], got["dwi"], got["dwo"]]
    for which in range(4):
      for trial in range(3):
        d = rng.standard_normal(base[which].shape)
        plus = [a + 1e-6 * d if i == which else a for i, a in enumerate(base)]
        minus = [a - 1e-6 * d if i == which else a for i, a in enumerate(base)]
        fd = (scalar(*plus) - scalar(*minus)) / 2e-6
        an = float((grads[which].astype(np.float64) * d).sum())
        assert abs(fd - an) <= 2e-4 * max(1.0, abs(fd)), (which, trial, fd, an)
    return
  if perturb == "sample":       # sampled experts differ from the arg-max
    assert (aux["index_1"] != aux["logits"].argmax(-1)).any()
  elif perturb:
    mult = aux["gate_mult"].astype(np.float64).reshape(b, l, m)
    assert np.abs(mult - 1).max() > 0.05
  assert not (aux["kept_1"] | aux["kept_2"]).all()     # drops are exercised
  if gating == "ntlb":
    assert (aux["taken_in_pass"] > 0).any()        # tokens placed by a later choice
  m1 = (nonpad.reshape(aux["kept_1"].shape) == 1).astype(np.float64)
  z = hp.moe_z_loss if gating == "switch" else None
  density_2 = None
  if loss2:
    # counted before the second-choice policy, which drops some of them here
    m2 = (nonpad.reshape(aux["kept_1"].shape) > 0)
    assert (m2 & ~aux["kept_2"]).any()
    density_2 = ((aux["index_2"][..., None] == np.arange(e))
                 * m2[..., None]).mean(1)

  def scalar(xv, wgv, wiv, wov):
    out, loss = _f64_layer(xv.reshape(b, l, m), wgv, wiv, wov, aux, gating, m1,
                           0.5, mb, z, mult, hnoise, density_2, activation)
    return (out * d_out.reshape(out.shape)).sum() + d_loss * loss
  base = [np.asarray(a).astype(np.float64)
          for a in (x.reshape(b, l, m), wg, wi, wo)]
  grads = [got["dx"].reshape(b, l, m), got["dw_gate"], got["dwi"], got["dwo"]]
  if isinstance(activation, list):
    # the kernels of the factors, stacked: one perturbation moves all of them
    grads[2] = np.stack(got["dwi"])
    inner = scalar
    scalar = lambda xv, wgv, wiv, wov: inner(xv, wgv, list(wiv), wov)
  eps = 1e-6
  for which in range(4):
    for trial in range(3):
      d = rng.standard_normal(base[which].shape)
      plus = [a + eps * d if i == which else a for i, a in enumerate(base)]
      minus = [a - eps * d if i == which else a for i, a in enumerate(base)]
      fd = (scalar(*plus) - scalar(*minus)) / (2 * eps)
      an = float((grads[which].astype(np.float64) * d).sum())
      assert abs(fd - an) <= 2e-4 * max(1.0, abs(fd)), (which, trial, fd, an)


def _f64_layer_v2(x, w_outer, w_inner, wi, wo, aux, m1_outer, coef, mb):
  """Independent float64 forward of the hierarchical layer with the routing of
  BOTH levels held fixed (experts, kept masks, slots, inner importance and
  density counts from `aux`), written per (token, choice) pair."""
  rx, ry = aux["outer"], aux["inner"]
  ag, s = rx["kept_1"].shape
  x_e, y_e = w_inner.shape[0], w_inner.shape[2]
  c = aux["capacity_x"]
  h0, t_ = aux["groups_y"]
  imp_in = (aux["importance_inner"].reshape(x_e * h0, t_) == 1).astype(np.float64)

  def gates(p, i1, i2, m1, k1, k2):
    g1 = p[i1] * m1
    g2 = p[i2] * (1.0 - (i2 == i1) * m1)
    den = g1 + g2 + 1e-9
    return g1 / den * k1, g2 / den * k2

  n = wo.shape[-1]
  out = np.zeros((ag, s, n))
  px = scipy.special.softmax(x @ w_outer, axis=-1)               # [ag,s,X]
  py_sum = np.zeros((x_e * h0, y_e))                             # inner proxy
  for gi in range(ag):
    for si in range(s):
      gx = gates(px[gi, si], rx["index_1"][gi, si], rx["index_2"][gi, si],
                 m1_outer[gi, si], float(rx["kept_1"][gi, si]),
                 float(rx["kept_2"][gi, si]))
      for k in range(2):
        if not rx["kept_%d" % (k + 1)][gi, si]:
          continue
        xe = int(rx["index_%d" % (k + 1)][gi, si])
        slot = gi * c + int(rx["pos_%d" % (k + 1)][gi, si])      # in [0, ag*c)
        hh, tt = divmod(slot, t_)
        row = xe * h0 + hh
        v = x[gi, si]
        py = scipy.special.softmax(v @ w_inner[xe])
        py_sum[row] += py * imp_in[row, tt]
        gy = gates(py, ry["index_1"][row, tt], ry["index_2"][row, tt],
                   imp_in[row, tt], float(ry["kept_1"][row, tt]),
                   float(ry["kept_2"][row, tt]))
        acc = np.zeros(n)
        for kk in range(2):
          ye = int(ry["index_%d" % (kk + 1)][row, tt])
          acc += gy[kk] * (np.maximum(v @ wi[ye, xe], 0.0) @ wo[ye, xe])
        out[gi, si] += gx[k] * acc
  # losses with the density counts fixed
  e1 = (rx["index_1"][..., None] == np.arange(x_e)) * m1_outer[..., None]
  loss_x = ((px * m1_outer[..., None]).mean(1) * e1.mean(1)).mean() * x_e * x_e
  e2 = (ry["index_1"][..., None] == np.arange(y_e)) * imp_in[..., None]
  # empty outer slots hold zero rows: their softmax is uniform but their
  # importance is 0, so they add nothing to the inner proxy
  loss_y = ((py_sum / t_) * e2.mean(1)).mean() * y_e * y_e
  return out, (loss_x + loss_y) / mb * coef


def test_v2_backward_against_central_differences():
  rng = np.random.default_rng(62)
  b, l, m, h = 2, 16, 5, 7
  x_e, y_e = 2, 3
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  w_outer = rng.standard_normal((m, x_e)).astype(np.float32)
  w_inner = rng.standard_normal((x_e, m, y_e)).astype(np.float32)
  wi = (rng.standard_normal((y_e, x_e, m, h)) / 2).astype(np.float32)
  wo = (rng.standard_normal((y_e, x_e, h, m)) / 3).astype(np.float32)
  nonpad = (rng.random((b, l)) < 0.85).astype(np.float32)
  d_out = rng.standard_normal((b, l, m)).astype(np.float32)
  d_loss, mb = 1.3, 2
  hp = _hp(moe_num_experts=[x_e, y_e], moe_hidden_size=h, moe_group_size=16,
           moe_capacity_factor_train=1.5, moe_capacity_factor_second_level=1.0,
           moe_min_expert_capacity=2, moe_loss_coef=0.5)
  got = O.moe_layer_v2_backward(x, w_outer, w_inner, wi, wo, hp, True,
                                "float32", d_out, d_loss, nonpadding=nonpad,
                                num_microbatches=mb)
  aux = got["aux"]
  rx, ry = aux["outer"], aux["inner"]
  assert not (rx["kept_1"] | rx["kept_2"]).all() or not ry["kept_2"].all()
  ag, s = rx["kept_1"].shape
  m1 = (nonpad.reshape(ag, s) == 1).astype(np.float64)

  def scalar(xv, a, bq, cq, dq):
    out, loss = _f64_layer_v2(xv.reshape(ag, s, m), a, bq, cq, dq, aux, m1,
                              0.5, mb)
    return (out * d_out.reshape(out.shape)).sum() + d_loss * loss
  base = [a.astype(np.float64) for a in (x, w_outer, w_inner, wi, wo)]
  # the forward restatement itself (more than one outer expert) against the
  # independent float64 forward: output per token and the loss
  fwd_out, fwd_loss, _ = O.moe_layer_v2(x, w_outer, w_inner, wi, wo, hp, True,
                                        "float32", nonpadding=nonpad,
                                        num_microbatches=mb)
  ref_out, ref_loss = _f64_layer_v2(base[0].reshape(ag, s, m), *base[1:], aux,
                                    m1, 0.5, mb)
  assert np.abs(ref_out).max() > 0.1
  np.testing.assert_allclose(fwd_out.reshape(ref_out.shape), ref_out,
                             rtol=1e-5, atol=1e-5)
  np.testing.assert_allclose(fwd_loss, ref_loss, rtol=1e-5)
  grads = [got["dx"], got["dw_outer"], got["dw_inner"], got["dwi"], got["dwo"]]
  eps = 1e-6
  for which in range(5):
    for trial in range(2):
      d = rng.standard_normal(base[which].shape)
      plus = [a + eps * d if i == which else a for i, a in enumerate(base)]
      minus = [a - eps * d if i == which else a for i, a in enumerate(base)]
      fd = (scalar(*plus) - scalar(*minus)) / (2 * eps)
      an = float((grads[which].astype(np.float64) * d).sum())
      assert abs(fd - an) <= 1e-4 * max(1.0, abs(fd)), (which, trial, fd, an)


def test_gate_input_perturbations():
  """moe.py:1189-1199: the router (only) sees perturbed inputs while training.
  jitter eps = 0 and eval mode change nothing; dropout with every u below
  keep_prob scales the router's input, hence its logits, by 1 / keep_prob; the
  experts always see the unperturbed tokens."""
  rng = np.random.default_rng(77)
  b, l, m, h, e = 2, 32, 8, 12, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wg = rng.standard_normal((m, e)).astype(np.float32)
  wi = rng.standard_normal((e, m, h)).astype(np.float32) / 3
  wo = rng.standard_normal((e, h, m)).astype(np.float32) / 3
  noise = rng.random((b, l, m)).astype(np.float32)
  kw = dict(moe_gating="switch", moe_num_experts=e, moe_hidden_size=h,
            moe_group_size=32, moe_switch_policy_eval="input_jitter")
  base = O.moe_layer_v1(x, wg, wi, wo, _hp(moe_switch_policy_train="argmax", **kw),
                        True, dense=False)
  same = O.moe_layer_v1(x, wg, wi, wo,
                        _hp(moe_switch_policy_train="input_jitter",
                            moe_switch_jitter=0.0, **kw), True, dense=False,
                        gate_noise=noise)
  np.testing.assert_array_equal(base[0], same[0])
  ev = O.moe_layer_v1(x, wg, wi, wo,
                      _hp(moe_switch_policy_train="input_jitter", **kw), False,
                      dense=False)                    # eval: no noise needed
  assert ev[2]["gate_mult"] is None
  jit = O.moe_layer_v1(x, wg, wi, wo,
                       _hp(moe_switch_policy_train="input_jitter",
                           moe_switch_jitter=0.5, **kw), True, dense=False,
                       gate_noise=noise)
  mult = jit[2]["gate_mult"]
  assert mult.min() >= 0.5 and mult.max() < 1.5
  np.testing.assert_allclose(jit[2]["logits"].reshape(b, l, e),
                             (x.astype(np.float64) * mult.reshape(b, l, m)) @ wg,
                             rtol=1e-5, atol=1e-5)
  np.testing.assert_array_equal(                       # experts see x itself
      jit[2]["expert_in"][jit[2]["index_1"][0, 0], 0, jit[2]["pos_1"][0, 0]]
      if jit[2]["kept_1"][0, 0] else x[0, 0], x[0, 0])
  drop = O.moe_layer_v1(x, wg, wi, wo,
                        _hp(moe_switch_policy_train="input_dropout",
                            moe_switch_dropout=0.2, **kw), True, dense=False,
                        gate_noise=np.zeros_like(noise))
  np.testing.assert_allclose(drop[2]["logits"], base[2]["logits"] / 0.8,
                             rtol=1e-5, atol=1e-6)
  with pytest.raises(NotImplementedError, match="gate_noise"):
    O.moe_layer_v1(x, wg, wi, wo,
                   _hp(moe_switch_policy_train="input_jitter", **kw), True)


def test_switch_sample_policy():
  """moe.py:1213-1216 with ops.py:5070-5086: the expert is the arg-max of
  logits + Gumbel(u) * temperature, the gate the softmax probability of that
  expert.  Temperature 0 is the arg-max policy; u -> 1 at one expert (a huge
  Gumbel value) forces that expert."""
  rng = np.random.default_rng(88)
  g, s, e, c = 2, 40, 5, 100
  logits = rng.standard_normal((g, s, e)).astype(np.float32)
  u = rng.random((g, s, e)).astype(np.float32)
  np.testing.assert_array_equal(O.sample_choice_logits(logits, 0.0, u), logits)
  ch = O.sample_choice_logits(logits, 1.5, u)
  u64 = 1e-9 + u.astype(np.float64) * (1 - 1e-9)
  np.testing.assert_allclose(ch, logits - 1.5 * np.log(-np.log(u64)),
                             rtol=1e-4, atol=1e-4)   # float32 logs of u near 1
  forced = np.full((g, s, e), 0.5, np.float32)
  target = rng.integers(0, e, size=(g, s))
  np.put_along_axis(forced, target[..., None], np.float32(1 - 1e-7), -1)
  r = O.switch_gating(logits, c,
                      choice_logits=O.sample_choice_logits(logits, 50.0, forced))
  np.testing.assert_array_equal(r["index_1"], target)
  p = scipy.special.softmax(logits.astype(np.float64), -1)
  np.testing.assert_allclose(
      r["gate_1"], np.take_along_axis(p, target[..., None], -1)[..., 0],
      rtol=2e-6)
  # the loss counts the sampled experts
  dens = (target[..., None] == np.arange(e)).mean(1)
  np.testing.assert_allclose(r["loss"], e * e * (p.mean(1) * dens).mean(),
                             rtol=1e-5)
  rm = O.switch_max_gating(logits, s, choice_logits=O.sample_choice_logits(
      logits, 50.0, forced))
  np.testing.assert_array_equal(rm["index_1"], target)


# ---- training-time summaries of the f1 routers ------------------------------
def test_router_summaries_closed_forms():
  """Uniform logits: every row's entropy is log E (up to the 1e-9 inside the
  log), the largest probability 1 / E, the arg-max always expert 0, the z-loss
  (c + log E)^2 / microbatches; S tokens on one expert with capacity C:
  fraction_routed = C / S.  Rows that are one-hot after the softmax: entropy
  0, gate 1."""
  g, s, e, c = 2, 16, 4, 5
  lg = np.full((g, s, e), 0.75, np.float32)
  r = O.switch_gating(lg, c)
  out = O.router_summaries(lg, "switch", r, num_microbatches=2)
  np.testing.assert_allclose(out["entropy"], np.log(e), rtol=1e-6)
  np.testing.assert_allclose(out["expert_gate"], 1.0 / e, rtol=1e-6)
  np.testing.assert_array_equal(out["experts"], [1, 0, 0, 0])
  np.testing.assert_allclose(out["fraction_routed"], c / s, rtol=1e-6)
  np.testing.assert_allclose(out["z_loss"], (0.75 + np.log(e)) ** 2 / 2,
                             rtol=1e-6)
  # importance: tokens that are not 1 leave the expert counts and the z-loss,
  # fraction_routed divides by the SUM of importance (moe.py:1286-1289)
  imp = np.ones((g, s), np.float32)
  imp[:, ::2] = 0.5
  r = O.switch_gating(lg, c, importance=imp)
  out = O.router_summaries(lg, "switch", r, importance=imp, num_microbatches=1)
  np.testing.assert_allclose(out["fraction_routed"],
                             r["kept_1"].sum() / imp.sum(), rtol=1e-6)
  np.testing.assert_allclose(out["z_loss"], (0.75 + np.log(e)) ** 2, rtol=1e-6)
  sharp = np.zeros((1, 8, 4), np.float32)
  sharp[0, np.arange(8), np.arange(8) % 4] = 60.0
  r = O.switch_gating(sharp, 8)
  out = O.router_summaries(sharp, "switch", r)
  assert abs(float(out["entropy"])) < 1e-6
  np.testing.assert_allclose(out["expert_gate"], 1.0, rtol=1e-6)
  np.testing.assert_allclose(out["experts"], [0.25] * 4)
  np.testing.assert_allclose(out["fraction_routed"], 1.0)


@pytest.mark.parametrize("gating", ["switch", "switch_max", "ntlb"])
def test_router_summaries_against_per_token_loop(gating):
  rng = np.random.default_rng(77)
  g, s, e, c, k = 3, 40, 6, 9, 3
  lg = (rng.standard_normal((g, s, e)) * 2).astype(np.float32)
  imp = rng.choice(np.array([0.0, 0.5, 1.0], np.float32), size=(g, s),
                   p=[0.2, 0.1, 0.7])
  if gating == "switch":
    r = O.switch_gating(lg, c, importance=imp)
  elif gating == "switch_max":
    r = O.switch_max_gating(lg, c, importance=imp)
  else:
    r = O.ntlb_gating(lg, c, k, importance=imp)
  out = O.router_summaries(lg, gating, r, importance=imp, top_k=k,
                           num_microbatches=2)
  p = scipy.special.softmax(lg.astype(np.float64), axis=-1)
  ent, gate, counts, lse2, ones = 0.0, 0.0, np.zeros(e), 0.0, 0
  for gi in range(g):
    for si in range(s):
      row = p[gi, si]
      ent += float(-(row * np.log(row + 1e-9)).sum())
      order = sorted(range(e), key=lambda j: (-row[j], j))
      gate += row[order[0]]
      if imp[gi, si] == 1.0:
        ones += 1
        lse2 += float(scipy.special.logsumexp(lg[gi, si].astype(np.float64))) ** 2
        for j in order[:k if gating == "ntlb" else 1]:
          counts[j] += 1
  np.testing.assert_allclose(out["entropy"], ent / (g * s), rtol=1e-5)
  np.testing.assert_allclose(out["expert_gate"], gate / (g * s), rtol=1e-5)
  np.testing.assert_allclose(out["experts"], counts / counts.sum(), rtol=1e-6)
  if gating != "ntlb":
    np.testing.assert_allclose(out["z_loss"], lse2 / (ones * 2), rtol=1e-5)
    np.testing.assert_allclose(out["fraction_routed"],
                               r["kept_1"].sum() / imp.sum(), rtol=1e-6)
    assert 0 < out["fraction_routed"] < 1


def test_router_summaries_expert_selection():
  """Column softmax: uniform logits over S unmasked tokens give entropy log S
  per (group, expert); every slot names one token, so group_token sums to
  G * E * C times the factor E * C the reference multiplies in
  (moe.py:1155-1158); against a float64 loop on random logits."""
  g, s, e, c = 2, 12, 3, 4
  imp = np.ones((g, s), np.float32)
  lg = np.zeros((g, s, e), np.float32)
  r = O.expert_selection_gating(lg, c, imp)
  out = O.router_summaries(lg, "expert_selection", r, importance=imp)
  np.testing.assert_allclose(out["entropy"], np.log(s), rtol=1e-6)
  np.testing.assert_allclose(out["group_token"].sum(), g * e * c * e * c)
  # ties go to the lowest tokens: every expert of every group takes 0..c-1
  np.testing.assert_array_equal(out["group_token"][:c], [g * e * e * c] * c)
  rng = np.random.default_rng(5)
  lg = (rng.standard_normal((g, s, e)) * 2).astype(np.float32)
  imp[:, -3:] = 0.0
  r = O.expert_selection_gating(lg, c, imp)
  out = O.router_summaries(lg, "expert_selection", r, importance=imp)
  x = lg.astype(np.float64) + (imp == 0)[..., None] * -1e9
  p = scipy.special.softmax(x, axis=1)
  np.testing.assert_allclose(out["entropy"],
                             (-(p * np.log(p + 1e-9)).sum(1)).mean(), rtol=1e-5)
  assert out["group_token"][-3:].sum() == 0           # masked tokens are never taken
