"""Shared input generators and comparison helpers for the tests."""

import numpy as np
import torch

from oracle import moe_oracle as O

ACT_TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def to_gpu(a, act_dtype="float32"):
  """float32 NumPy array holding activation-dtype values -> GPU tensor."""
  t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
  return t.to(ACT_TORCH[act_dtype]).cuda().contiguous()


def to_np(t):
  return t.detach().float().cpu().numpy()


def random_logits(rng, g, s, e, scale=1.0, quantum=None):
  x = rng.standard_normal((g, s, e)).astype(np.float32) * np.float32(scale)
  if quantum:
    x = (np.round(x / quantum) * quantum).astype(np.float32)
  return x


def safe_logits(rng, g, s, e, scale=1.0, bias=None, min_gap=1e-4, top=3):
  """Random logits whose `top` largest entries per row differ by at least
  `min_gap` (rows that do not are redrawn), so that the choice of the first
  top - 1 experts does not depend on the last ulps of exp/log."""
  x = random_logits(rng, g, s, e, scale)
  if bias is not None:
    x = x + bias
  k = min(top, e)
  for _ in range(100):
    best = -np.sort(-x, axis=-1)[..., :k]
    bad = ((best[..., :-1] - best[..., 1:]) < min_gap).any(axis=-1)
    if not bad.any():
      return x
    fresh = random_logits(rng, 1, int(bad.sum()), e, scale)[0]
    if bias is not None:
      fresh = fresh + bias
    x[bad] = fresh
  raise AssertionError("could not separate the top logits")


def near_bf16_midpoint(v, margin):
  """True where |v| lies within `margin` bfloat16 ulps of the midpoint between
  two neighbouring bfloat16 values (where a last-bits difference between two
  float32 evaluations of v could round to different bfloat16 values)."""
  v = np.abs(np.asarray(v, np.float64))
  ok = v > 0
  scaled = np.where(ok, v, 1.0)
  scaled = scaled / 2.0 ** (np.floor(np.log2(scaled)) - 7)     # [128, 256)
  frac = scaled - np.floor(scaled)
  return ok & (np.abs(frac - 0.5) < margin)


def bf16_softmax_fragile_rows(x, ulps=8):
  """Rows of float32 logits x [..., E] on which the bfloat16 softmax of the
  ntlb router could come out differently in two correct implementations.  The
  additions of the chain are correctly rounded everywhere, so implementations
  can only part where an exp or log result lies within a few float32 ulps of a
  bfloat16 rounding midpoint (judged on the float64 result, `ulps` float32
  ulps either side).  Equal bfloat16 probabilities are fine: ties go by
  index on both sides."""
  from oracle import moe_oracle as O
  margin = ulps * 2.0 ** -16
  xb = O.round_bf16(x).astype(np.float64)
  m = xb.max(-1, keepdims=True)
  t = O.round_bf16((xb - m).astype(np.float32)).astype(np.float64)
  u64 = np.exp(t)
  bad = near_bf16_midpoint(u64, margin).any(-1)
  u = O.round_bf16(u64.astype(np.float32))
  sm = O.round_bf16(O.seq_sum(u, axis=-1)).astype(np.float64)
  l64 = np.log(sm)
  bad |= near_bf16_midpoint(l64, margin)
  lse = O.round_bf16((O.round_bf16(l64.astype(np.float32)).astype(np.float64)
                      + m[..., 0]).astype(np.float32)).astype(np.float64)
  d = O.round_bf16((xb - lse[..., None]).astype(np.float32)).astype(np.float64)
  bad |= near_bf16_midpoint(np.exp(d), margin).any(-1)
  return bad


def bf16_softmax_safe_logits(rng, g, s, e, scale=1.0, bias=None, ulps=8):
  """Random logits [g, s, e] without rows that bf16_softmax_fragile_rows
  flags (those are redrawn)."""
  def draw(n):
    x = random_logits(rng, 1, n, e, scale)[0]
    return x if bias is None else x + bias

  x = draw(g * s).reshape(g, s, e)
  for _ in range(100):
    bad = bf16_softmax_fragile_rows(x, ulps)
    if not bad.any():
      return x
    x[bad] = draw(int(bad.sum()))
  raise AssertionError("could not find rows away from the rounding midpoints")


def min_relative_gap(p, k=3):
  """Smallest relative gap between consecutive members of the top-k of each
  softmax row: routing is only implementation-independent when this is well
  above a few float32 ulps."""
  top = -np.sort(-p, axis=-1)[..., :k]
  gaps = (top[..., :-1] - top[..., 1:]) / np.maximum(top[..., :-1], 1e-30)
  return float(gaps.min())


def zipf_bias(rng, e, scale=3.0, s=1.2):
  ranks = rng.permutation(e) + 1
  return (scale * ranks.astype(np.float64) ** (-s)).astype(np.float32)


def routing_to_np(r):
  """mesh_amd.moe_hip.Routing -> dict shaped like the oracle's record."""
  idx, pos = to_np(r.idx).astype(np.int32), to_np(r.pos).astype(np.int32)
  gate, kept = to_np(r.gate), to_np(r.kept) != 0
  return dict(index_1=idx[..., 0], index_2=idx[..., 1], pos_1=pos[..., 0],
              pos_2=pos[..., 1], gate_1=gate[..., 0], gate_2=gate[..., 1],
              kept_1=kept[..., 0], kept_2=kept[..., 1],
              fill=to_np(r.fill).astype(np.int32), loss=to_np(r.loss)[0])


def assert_routing_equal(got, want, gate_rtol=1e-5):
  """Bit-exact expert indices, positions, kept masks and fill counts; gates to
  float32 round-off."""
  for k in ("index_1", "index_2", "kept_1", "kept_2", "pos_1", "pos_2", "fill"):
    np.testing.assert_array_equal(got[k], want[k], err_msg=k)
  for k in ("gate_1", "gate_2"):
    np.testing.assert_allclose(got[k], want[k], rtol=gate_rtol, atol=1e-7,
                               err_msg=k)


def safe_tokens(rng, n_tok, m, w_gate, act_dtype, bias=None, min_gap=1e-3,
                ones_column=False, top=3, bf16_router=False):
  """x [n_tok, m] ~ N(0,1) in the activation dtype such that the router logits
  x . w_gate (+ bias) have their `top` largest entries per token at least
  `min_gap` apart (offending tokens are redrawn): the routing then does not
  depend on the summation order of the router matmul.  bf16_router (the ntlb
  router with bfloat16 activations, which rounds its logits to bfloat16 and
  runs its softmax there): instead, no logit of a token may sit within 2 % of
  a bfloat16 ulp of a rounding midpoint (two summation orders of the matmul
  then round it alike) and the row must not be one that
  bf16_softmax_fragile_rows flags."""
  wg = O.cast_act(w_gate, act_dtype)
  x = O.cast_act(rng.standard_normal((n_tok, m)).astype(np.float32), act_dtype)
  k = min(top, wg.shape[1])
  for _ in range(100):
    logits = O.router_logits(x, wg)
    if bias is not None:
      logits = logits + bias
    top = -np.sort(-logits, axis=-1)[..., :k]
    bad = ((top[..., :-1] - top[..., 1:]) < min_gap).any(axis=-1)
    if bf16_router:
      bad = (near_bf16_midpoint(logits, 0.02).any(axis=-1)
             | bf16_softmax_fragile_rows(logits))
    if not bad.any():
      return x
    x[bad] = O.cast_act(
        rng.standard_normal((int(bad.sum()), m)).astype(np.float32), act_dtype)
  raise AssertionError("could not separate the router logits")


def normal_weights(rng, shape, fan_in):
  return (rng.standard_normal(shape) / np.sqrt(fan_in)).astype(np.float32)


def value_tolerance(act_dtype):
  """Output tolerance of the layer: rtol 1e-4 for float32 (plus an absolute
  floor for entries that cancel to ~0), rtol 2e-2 / atol 1e-2 for bfloat16."""
  if act_dtype == "bfloat16":
    return dict(rtol=2e-2, atol=1e-2)
  return dict(rtol=1e-4, atol=2e-5)


def assert_routing_properties(r, logits, importance=None):
  """Size-independent properties of a top-2 Routing `r` (GPU tensors) computed
  from float32 `logits` [G, S, E] (GPU): what the definition of the capacity
  assignment (transformer/moe.py:1397-1496) fixes without running the oracle.
  importance [G, S] float32 with values in {0, 0.5, 1} or None.  Returns the
  boolean slot occupancy [G, E, C]."""
  g, s, e = logits.shape
  c = r.capacity
  dev = logits.device
  idx, pos, kept = r.idx.long(), r.pos.long(), r.kept.bool()
  # first / second expert: argmax and argmax-with-first-removed of the logits
  # (softmax is monotone; ties have measure zero for continuous random logits)
  top2 = logits.topk(2, dim=-1).indices
  if importance is None:
    assert torch.equal(idx, top2)
    competing = torch.ones((g, s, 2), dtype=torch.bool, device=dev)
  else:
    one = importance == 1.0
    half = (importance > 0) & ~one
    assert torch.equal(idx[one], top2[one])
    # 0 < importance < 1: the best expert, offered as a second choice
    assert torch.equal(idx[half][:, 1], top2[half][:, 0])
    competing = torch.stack([one, one | half], dim=-1)
    assert not bool(kept[~competing].any())
    assert not bool(r.gate[~competing].any())
  # every (group, expert) fills slots 0..fill-1 exactly once, fill <= C
  gi = torch.arange(g, device=dev).view(g, 1, 1).expand(g, s, 2)
  slot = (gi * e + idx) * c + pos
  used = torch.zeros(g * e * c, dtype=torch.int32, device=dev)
  used.scatter_add_(0, slot[kept], torch.ones_like(slot[kept], dtype=torch.int32))
  assert int(used.max()) <= 1
  used = used.view(g, e, c)
  fill = r.fill.long()
  assert int(fill.max()) <= c
  want_used = (torch.arange(c, device=dev).view(1, 1, c) < fill.unsqueeze(-1))
  assert torch.equal(used.bool(), want_used)
  assert torch.equal(used.sum(-1), fill)
  # kept <=> position below capacity, for every competing choice
  assert torch.equal(kept, (pos < c) & competing)
  # first choices of an expert precede its second choices
  first_count = torch.zeros(g * e, dtype=torch.long, device=dev)
  k1 = kept[..., 0]
  first_count.scatter_add_(0, (gi[..., 0] * e + idx[..., 0])[k1],
                           torch.ones(int(k1.sum()), dtype=torch.long,
                                      device=dev))
  c2 = competing[..., 1]
  key2 = (gi[..., 1] * e + idx[..., 1])
  assert bool((pos[..., 1] >= first_count[key2])[c2].all())
  first_second = torch.full((g * e,), 1 << 40, dtype=torch.long, device=dev)
  first_second.scatter_reduce_(0, key2[c2], pos[..., 1][c2], reduce="amin")
  has_second = first_second < (1 << 40)
  assert torch.equal(first_second[has_second], first_count[has_second])
  # positions grow by one per competing chooser, in token order, within
  # (group, expert, choice); choices that do not compete are set aside under
  # an expert id of their own
  for k in range(2):
    ek = torch.where(competing[..., k], idx[..., k], torch.full_like(idx[..., k], e))
    key = ek * s + torch.arange(s, device=dev).view(1, s)
    order = key.argsort(dim=1, stable=True)
    sorted_pos = pos[..., k].gather(1, order)
    sorted_e = ek.gather(1, order)
    same = (sorted_e[:, 1:] == sorted_e[:, :-1]) & (sorted_e[:, 1:] < e)
    assert bool(((sorted_pos[:, 1:] - sorted_pos[:, :-1])[same] == 1).all())
  # gates: the normalised pair sums to one where both are kept
  both = kept.all(-1)
  assert torch.allclose(r.gate.sum(-1)[both], torch.ones((), device=dev),
                        atol=1e-5)
  return want_used
