"""Pins of oracle/block_oracle.py: float64 closed forms, invariants and
hand-worked cases for the transformer block around the MoE layer."""

import numpy as np
import pytest
import scipy.special

from oracle import block_oracle as B
from oracle import moe_oracle as O


def test_rms_norm_against_float64():
  rng = np.random.default_rng(1)
  x = rng.standard_normal((3, 7, 48)).astype(np.float32) * 3
  scale = rng.standard_normal(48).astype(np.float32)
  x64 = x.astype(np.float64)
  want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * scale
  np.testing.assert_allclose(B.rms_norm(x, scale), want, rtol=2e-6, atol=1e-7)
  # a row of equal entries c normalises to sign(c) (eps aside)
  const = np.full((1, 16), -4.0, np.float32)
  np.testing.assert_allclose(B.rms_norm(const, np.ones(16, np.float32)),
                             -np.ones((1, 16)), rtol=1e-6)
  # scale-invariance: rms_norm(a x) = rms_norm(x) for a > 0 (eps negligible)
  np.testing.assert_allclose(B.rms_norm(8 * x, scale), B.rms_norm(x, scale),
                             rtol=1e-5, atol=1e-6)


def test_rms_norm_bf16_rounds_every_op():
  rng = np.random.default_rng(2)
  x = O.round_bf16(rng.standard_normal((5, 64)).astype(np.float32))
  scale = O.round_bf16(1 + 0.1 * rng.standard_normal(64).astype(np.float32))
  y = B.rms_norm(x, scale, "bfloat16")
  np.testing.assert_array_equal(y, O.round_bf16(y))
  x64 = x.astype(np.float64)
  want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * scale
  # six bf16 roundings in a row: within a few bf16 ulps of the exact value
  np.testing.assert_allclose(y, want, rtol=3e-2, atol=1e-3)


def test_dense_against_float64():
  rng = np.random.default_rng(3)
  x = rng.standard_normal((2, 9, 24)).astype(np.float32)
  w = rng.standard_normal((24, 40)).astype(np.float32)
  want = x.astype(np.float64) @ w.astype(np.float64)
  np.testing.assert_allclose(B.dense(x, w), want, rtol=1e-5, atol=1e-5)
  np.testing.assert_allclose(B.dense(x, w, activation="relu"),
                             np.maximum(want, 0), rtol=1e-5, atol=1e-5)


def _attention64(x, wq, wk, wv, wo, heads, causal):
  b, l, _ = x.shape
  d = wq.shape[1] // heads
  x, wq, wk, wv, wo = (a.astype(np.float64) for a in (x, wq, wk, wv, wo))
  out = np.zeros((b, l, wq.shape[1]))
  for bi in range(b):
    for h in range(heads):
      sl = slice(h * d, (h + 1) * d)
      q, k, v = x[bi] @ wq[:, sl], x[bi] @ wk[:, sl], x[bi] @ wv[:, sl]
      s = q @ k.T
      if causal:
        s = np.where(np.tril(np.ones((l, l), bool)), s, -np.inf)
      out[bi, :, sl] = scipy.special.softmax(s, axis=-1) @ v
  return out @ wo


@pytest.mark.parametrize("causal", [False, True])
def test_self_attention_against_float64(causal):
  rng = np.random.default_rng(4)
  b, l, m, heads, d = 2, 12, 16, 3, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wq, wk, wv = (rng.standard_normal((m, heads * d)).astype(np.float32) / 3
                for _ in range(3))
  wo = rng.standard_normal((heads * d, m)).astype(np.float32) / 3
  got = B.self_attention(x, wq, wk, wv, wo, heads, causal)
  np.testing.assert_allclose(got, _attention64(x, wq, wk, wv, wo, heads, causal),
                             rtol=2e-5, atol=2e-5)


def test_self_attention_causality_and_uniform_case():
  rng = np.random.default_rng(5)
  b, l, m, heads, d = 1, 10, 8, 2, 4
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  wq, wk, wv = (rng.standard_normal((m, heads * d)).astype(np.float32)
                for _ in range(3))
  wo = np.eye(heads * d, m, dtype=np.float32)
  base = B.self_attention(x, wq, wk, wv, wo, heads, True)
  x2 = x.copy()
  x2[:, 6:] = rng.standard_normal((b, 4, m))
  moved = B.self_attention(x2, wq, wk, wv, wo, heads, True)
  np.testing.assert_array_equal(base[:, :6], moved[:, :6])     # the past is fixed
  assert np.abs(base[:, 6:] - moved[:, 6:]).max() > 1e-3
  full = B.self_attention(x2, wq, wk, wv, wo, heads, False)
  assert np.abs(full[:, :6] - base[:, :6]).max() > 1e-3         # not so unmasked
  # zero queries: uniform weights, output t = mean of the values 0..t
  out = B.self_attention(x, np.zeros_like(wq), wk, wv, wo, heads, True)
  v = x[0].astype(np.float64) @ wv.astype(np.float64)
  want = np.cumsum(v, axis=0) / np.arange(1, l + 1)[:, None]
  np.testing.assert_allclose(out[0], want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_sequence_ids_are_block_diagonal(causal):
  """With sequence ids over contiguous segments, attention over the packed row
  equals attention over every segment on its own (what "a query sees only its
  own sequence" means, transformer_layers.py:303-316), forward and backward."""
  rng = np.random.default_rng(77 + causal)
  b, l, heads, d = 2, 24, 2, 4
  ids = np.array([[1] * 7 + [2] * 9 + [3] * 5 + [0] * 3,
                  [5] * 12 + [6] * 12], np.int32)
  q, k, v, do = (rng.standard_normal((b, l, heads * d)).astype(np.float32)
                 for _ in range(4))
  got = B._attention_core(q, k, v, heads, causal, "float32", sequence_id=ids)
  got_b = B.attention_core_backward(q, k, v, do, heads, causal, "float32",
                                    sequence_id=ids)
  for i in range(b):
    for sid in np.unique(ids[i]):
      seg = np.nonzero(ids[i] == sid)[0]
      sl = slice(seg[0], seg[-1] + 1)
      part = lambda t: t[i:i + 1, sl]
      want = B._attention_core(part(q), part(k), part(v), heads, causal,
                               "float32")
      np.testing.assert_allclose(got[i:i + 1, sl], want, rtol=1e-5, atol=1e-6)
      want_b = B.attention_core_backward(part(q), part(k), part(v), part(do),
                                         heads, causal, "float32")
      for g_, w_ in zip(got_b, want_b):
        np.testing.assert_allclose(g_[i:i + 1, sl], w_, rtol=1e-5, atol=1e-6)


def test_attention_incremental_is_a_row_of_causal_attention():
  """A decoding step at position p gives row p of the autoregressive attention
  over the full row, whatever the states hold at and after p; the step's key
  and value land in row p of the new states and nothing else moves."""
  rng = np.random.default_rng(78)
  b, l, heads, d = 2, 12, 2, 4
  q, k, v = (rng.standard_normal((b, l, heads * d)).astype(np.float32)
             for _ in range(3))
  full = B._attention_core(q, k, v, heads, True, "float32")
  values = rng.standard_normal((heads, 8)).astype(np.float32)
  full_rel = B._attention_core(q, k, v, heads, True, "float32",
                               relative_values=values)
  assert np.abs(full - full_rel).max() > 1e-2
  for p in ([0, 0], [5, 9], [11, 3]):
    kc, vc = k.copy(), v.copy()
    for i, pi in enumerate(p):
      kc[i, pi:] = 7.0
      vc[i, pi:] = -3.0
    rows = np.arange(b)
    out, k2, v2 = B.attention_incremental(q[rows, p], k[rows, p], v[rows, p], kc,
                                          vc, np.array(p), heads)
    np.testing.assert_allclose(out, full[rows, p], rtol=1e-5, atol=1e-6)
    # the same with a relative attention bias
    out_rel = B.attention_incremental(q[rows, p], k[rows, p], v[rows, p], kc, vc,
                                      np.array(p), heads,
                                      relative_values=values)[0]
    np.testing.assert_allclose(out_rel, full_rel[rows, p], rtol=1e-5, atol=1e-6)
    for i, pi in enumerate(p):
      np.testing.assert_array_equal(k2[i, :pi + 1], k[i, :pi + 1])
      np.testing.assert_array_equal(v2[i, :pi + 1], v[i, :pi + 1])
      np.testing.assert_array_equal(k2[i, pi + 1:], kc[i, pi + 1:])


def test_relative_position_bucket_known_values():
  """The bucket rule by its definition (transformer_layers.py:1000-1042): half
  of the range exact, the other half logarithmic up to max_distance, positive
  relative positions in the upper half when bidirectional, invisible (clamped
  to 0) when not."""
  rp = B.relative_position_bucket
  # bidirectional, 32 buckets: 16 per direction, 8 exact
  assert list(rp(np.arange(0, -8, -1))) == list(range(8))
  assert list(rp(np.arange(0, 8))) == [0] + list(range(17, 24))
  assert rp(np.array(-8)) == 8 and rp(np.array(8)) == 24
  assert rp(np.array(-127)) == 15 and rp(np.array(-128)) == 15
  assert rp(np.array(-100000)) == 15 and rp(np.array(100000)) == 31
  # boundaries of the logarithmic half: n = 8 * 16^(i/8) enters bucket 8 + i
  for i in range(1, 8):
    edge = 8.0 * 16.0 ** (i / 8.0)
    lo, hi = int(np.floor(edge - 1e-9)), int(np.ceil(edge + 1e-9))
    if lo != hi:        # the edge itself is not an integer: no rounding doubt
      assert rp(np.array(-lo)) == 8 + i - 1 and rp(np.array(-hi)) == 8 + i
  # unidirectional: 16 exact, positive relative positions count as 0
  assert list(rp(np.arange(0, -16, -1), bidirectional=False)) == list(range(16))
  assert list(rp(np.arange(1, 5), bidirectional=False)) == [0, 0, 0, 0]
  assert rp(np.array(-16), False) == 16 and rp(np.array(-127), False) == 31
  got = rp(np.arange(0, -300, -1), bidirectional=False)
  assert (np.diff(got) >= 0).all() and got.max() == 31
  # the bias is a function of (memory position - query position) only
  values = np.arange(2 * 32, dtype=np.float32).reshape(2, 32)
  bias = B.relative_attention_bias(values, 20, True)
  assert bias.shape == (1, 2, 20, 20)
  for off in (-19, -3, 0, 5, 19):
    diag = np.diagonal(bias[0, 1], offset=off)
    assert (diag == diag[0]).all()
    assert diag[0] == values[1, rp(np.array(off))]


def test_relative_bias_gradient_against_finite_differences():
  rng = np.random.default_rng(79)
  b, l, heads, d, nb = 2, 10, 2, 4, 8
  q, k, v, do = (rng.standard_normal((b, l, heads * d)) for _ in range(4))
  values = rng.standard_normal((heads, nb))

  def f(vals):
    pos = np.arange(l)
    bucket = B.relative_position_bucket(pos[None, :] - pos[:, None], False, nb)
    q4, k4, v4 = (t.reshape(b, l, heads, d) for t in (q, k, v))
    logits = np.einsum("blhd,bmhd->bhlm", q4, k4) + vals[:, bucket][None]
    logits = logits + (pos[None, :] > pos[:, None]) * -1e9
    w = scipy.special.softmax(logits, axis=-1)
    out = np.einsum("bhlm,bmhd->blhd", w, v4).reshape(b, l, heads * d)
    return (out * do).sum()
  got = B.attention_core_backward(
      q.astype(np.float32), k.astype(np.float32), v.astype(np.float32),
      do.astype(np.float32), heads, True, "float32",
      relative_values=values.astype(np.float32))[3]
  want = np.zeros_like(values)
  eps = 1e-5
  for h in range(heads):
    for j in range(nb):
      up, dn = values.copy(), values.copy()
      up[h, j] += eps
      dn[h, j] -= eps
      want[h, j] = (f(up) - f(dn)) / (2 * eps)
  np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-4)


def test_self_attention_bf16_close_to_float32():
  rng = np.random.default_rng(6)
  b, l, m, heads, d = 2, 16, 32, 2, 8
  x = O.round_bf16(rng.standard_normal((b, l, m)).astype(np.float32))
  ws = [O.round_bf16(rng.standard_normal(s).astype(np.float32) / 5)
        for s in ((m, heads * d),) * 3 + ((heads * d, m),)]
  a = B.self_attention(x, *ws, heads, True, "bfloat16")
  np.testing.assert_array_equal(a, O.round_bf16(a))
  f = B.self_attention(x, *ws, heads, True, "float32")
  np.testing.assert_allclose(a, f, rtol=5e-2, atol=5e-2)


def _stack_weights(rng, m, e, hdim, heads, d):
  def n(*shape):
    return (rng.standard_normal(shape) / np.sqrt(shape[-2])).astype(np.float32)
  att = dict(kind="attention", num_heads=heads, wq=n(m, heads * d),
             wk=n(m, heads * d), wv=n(m, heads * d), wo=n(heads * d, m),
             scale=(1 + 0.1 * rng.standard_normal(m)).astype(np.float32))
  hp = O.default_hparams(moe_num_experts=e, moe_hidden_size=hdim,
                         moe_group_size=16, moe_second_policy_eval="all",
                         moe_capacity_factor_eval=2.0)
  moe = dict(kind="moe", w_gate=n(m, e), wi=n(e, m, hdim), wo=n(e, hdim, m),
             hparams=hp,
             scale=(1 + 0.1 * rng.standard_normal(m)).astype(np.float32))
  ffn = dict(kind="dense_relu_dense", wi=n(m, hdim), wo=n(hdim, m),
             scale=(1 + 0.1 * rng.standard_normal(m)).astype(np.float32))
  return [att, moe, dict(att), ffn]


def test_layer_stack_by_hand_and_zero_kernels():
  rng = np.random.default_rng(7)
  b, l, m = 2, 16, 24
  layers = _stack_weights(rng, m, 4, 32, 2, 8)
  final = (1 + 0.1 * rng.standard_normal(m)).astype(np.float32)
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  y, losses = B.layer_stack(x, layers, final, autoregressive=True)
  assert len(losses) == 1 and y.shape == x.shape
  # by hand: chain the pieces
  h = x
  a = layers[0]
  h = h + B.self_attention(B.rms_norm(h, a["scale"]), a["wq"], a["wk"], a["wv"],
                           a["wo"], 2, True)
  mo = layers[1]
  out, loss, _ = O.moe_layer_v1(B.rms_norm(h, mo["scale"]), mo["w_gate"],
                                mo["wi"], mo["wo"], mo["hparams"], False,
                                dense=False)
  h = h + out
  a = layers[2]
  h = h + B.self_attention(B.rms_norm(h, a["scale"]), a["wq"], a["wk"], a["wv"],
                           a["wo"], 2, True)
  f = layers[3]
  h = h + B.dense_relu_dense(B.rms_norm(h, f["scale"]), f["wi"], f["wo"])
  np.testing.assert_allclose(y, B.rms_norm(h, final), rtol=1e-6, atol=1e-6)
  assert losses[0] == loss
  # all output kernels zero: every layer adds 0 and the stack is its final norm
  zeroed = []
  for layer in layers:
    z = dict(layer)
    z["wo"] = np.zeros_like(layer["wo"])
    zeroed.append(z)
  y0, _ = B.layer_stack(x, zeroed, final)
  np.testing.assert_array_equal(y0, B.rms_norm(x, final))


def test_layer_stack_sequence_ids_by_hand():
  """Where the padding mask sits (transformer.py:462-489, :424): on every
  layer's input after its norm and on the stack's output, not on the residual
  stream; the experts get nonpadding as importance."""
  rng = np.random.default_rng(8)
  b, l, m = 2, 16, 24
  layers = _stack_weights(rng, m, 4, 32, 2, 8)
  final = (1 + 0.1 * rng.standard_normal(m)).astype(np.float32)
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  ids = np.array([[1] * 6 + [2] * 7 + [0] * 3, [3] * 16], np.int32)
  npad = (ids != 0).astype(np.float32)
  y, losses = B.layer_stack(x, layers, final, autoregressive=True,
                            sequence_id=ids)
  h = x
  a = layers[0]
  h = h + B.self_attention(B.rms_norm(h, a["scale"]) * npad[..., None], a["wq"],
                           a["wk"], a["wv"], a["wo"], 2, True, sequence_id=ids)
  mo = layers[1]
  out, loss, _ = O.moe_layer_v1(B.rms_norm(h, mo["scale"]) * npad[..., None],
                                mo["w_gate"], mo["wi"], mo["wo"], mo["hparams"],
                                False, nonpadding=npad, dense=False)
  h = h + out
  a = layers[2]
  h = h + B.self_attention(B.rms_norm(h, a["scale"]) * npad[..., None], a["wq"],
                           a["wk"], a["wv"], a["wo"], 2, True, sequence_id=ids)
  f = layers[3]
  h = h + B.dense_relu_dense(B.rms_norm(h, f["scale"]) * npad[..., None],
                             f["wi"], f["wo"])
  np.testing.assert_allclose(y, B.rms_norm(h, final) * npad[..., None],
                             rtol=1e-6, atol=1e-6)
  assert losses[0] == loss
  assert not y[0, -3:].any() and np.abs(h[0, -3:]).min() > 0


def test_dropout_noise_arguments():
  """The dropout hooks of the block oracle: noise of ones changes nothing; the
  product against float64; noise on the attention weights (what the reference
  does) equals noise on the values (what the fused kernel is given)."""
  rng = np.random.default_rng(9)
  b, l, m, heads, d, hid = 2, 10, 16, 2, 4, 12
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  noise = O.hidden_dropout_noise(rng.random((b, m)), 0.75, "float32")
  assert set(np.unique(noise)) == {np.float32(0), np.float32(1 / 0.75)}
  got = B.broadcast_dropout(x, noise, -2)
  np.testing.assert_allclose(got, x.astype(np.float64) * noise[:, None, :],
                             rtol=1e-6)
  assert (got[:, :, noise[0] == 0][0] == 0).all()
  np.testing.assert_array_equal(B.broadcast_dropout(x, np.ones((b, m)), -2), x)
  # bf16: threshold and quotient are bf16 scalars
  nb = O.hidden_dropout_noise(rng.random((b, m)), 0.9, "bfloat16")
  assert set(np.unique(nb)) <= {np.float32(0), np.float32(1.109375)}
  wq, wk, wv = (rng.standard_normal((m, heads * d)).astype(np.float32) / 3
                for _ in range(3))
  wo = rng.standard_normal((heads * d, m)).astype(np.float32) / 3
  ones = np.ones((b, heads, l), np.float32)
  np.testing.assert_array_equal(
      B.self_attention(x, wq, wk, wv, wo, heads, True, weights_noise=ones),
      B.self_attention(x, wq, wk, wv, wo, heads, True))
  wn = O.hidden_dropout_noise(rng.random((b, heads, l)), 0.6, "float32")
  got = B.self_attention(x, wq, wk, wv, wo, heads, False, weights_noise=wn)
  # float64, with the noise on the values instead: v[b, k, h, :] * noise[b, h, k]
  x64 = x.astype(np.float64)
  want = np.zeros((b, l, heads * d))
  for bi in range(b):
    for h in range(heads):
      sl = slice(h * d, (h + 1) * d)
      q, k, v = x64[bi] @ wq[:, sl], x64[bi] @ wk[:, sl], x64[bi] @ wv[:, sl]
      want[bi, :, sl] = scipy.special.softmax(q @ k.T, axis=-1) @ (
          v * wn[bi, h][:, None])
  np.testing.assert_allclose(got, want @ wo.astype(np.float64), rtol=2e-5,
                             atol=2e-5)
  wi = rng.standard_normal((m, hid)).astype(np.float32) / 4
  wo2 = rng.standard_normal((hid, m)).astype(np.float32) / 4
  hn = O.hidden_dropout_noise(rng.random((b, hid)), 0.5, "float32")
  got = B.dense_relu_dense(x, wi, wo2, hidden_noise=hn)
  want = (np.maximum(x64 @ wi, 0) * hn[:, None, :]) @ wo2
  np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)
  # the stack: by hand with one dense layer
  scale = np.ones(m, np.float32)
  layer = dict(kind="dense_relu_dense", scale=scale, wi=wi, wo=wo2,
               hidden_noise=hn, sublayer_noise=noise)
  first = O.hidden_dropout_noise(rng.random((b, m)), 0.8, "float32")
  last = O.hidden_dropout_noise(rng.random((b, m)), 0.8, "float32")
  y, _ = B.layer_stack(x, [layer], scale, initial_noise=first, final_noise=last)
  h = B.broadcast_dropout(x, first, -2)
  h = h + B.broadcast_dropout(
      B.dense_relu_dense(B.rms_norm(h, scale), wi, wo2, hidden_noise=hn),
      noise, -2)
  np.testing.assert_allclose(
      y, B.broadcast_dropout(B.rms_norm(h, scale), last, -2), rtol=1e-6,
      atol=1e-6)


def _fd(fn, arg, direction, eps=1e-6):
  """Central difference of the scalar fn along `direction` in float64."""
  return (fn(arg + eps * direction) - fn(arg - eps * direction)) / (2 * eps)


def test_backward_passes_against_float64_finite_differences():
  """Each backward restatement against central differences of a float64
  forward: <grad, direction> = d/dt loss(arg + t direction)."""
  rng = np.random.default_rng(11)
  b, l, m, heads, d = 2, 7, 12, 3, 4
  f64 = lambda *s: rng.standard_normal(s)
  x, dy, scale = f64(b, l, m), f64(b, l, m), 1 + 0.3 * f64(m)

  def rms64(x_, s_):
    return x_ / np.sqrt((x_ * x_).mean(-1, keepdims=True) + 1e-6) * s_
  dx, ds = B.rms_norm_backward(x, scale, dy)
  u, us = f64(b, l, m), f64(m)
  np.testing.assert_allclose(
      (dx * u).sum(), _fd(lambda a: (rms64(a, scale) * dy).sum(), x, u),
      rtol=2e-4)
  np.testing.assert_allclose(
      (ds * us).sum(), _fd(lambda s_: (rms64(x, s_) * dy).sum(), scale, us),
      rtol=2e-4)
  # a dropped mean term would leave dx with a component along x
  np.testing.assert_allclose(
      (B.rms_norm_backward(x, np.ones(m), x)[0]), 0, atol=2e-5)

  w, dyn = f64(m, 9) / 3, f64(b, l, 9)
  for act in (None, "relu"):
    fwd = lambda x_, w_: (np.maximum(x_ @ w_, 0) if act else x_ @ w_)
    dxd, dw = B.dense_backward(x, w, dyn, activation=act)
    uw = f64(m, 9)
    np.testing.assert_allclose(
        (dxd * u).sum(), _fd(lambda a: (fwd(a, w) * dyn).sum(), x, u),
        rtol=2e-4)
    np.testing.assert_allclose(
        (dw * uw).sum(), _fd(lambda a: (fwd(x, a) * dyn).sum(), w, uw),
        rtol=2e-4)

  q, k, v, do = (f64(b, l, heads * d) for _ in range(4))

  def core64(q_, k_, v_, causal):
    out = np.zeros((b, l, heads * d))
    for bi in range(b):
      for h in range(heads):
        sl = slice(h * d, (h + 1) * d)
        s = q_[bi, :, sl] @ k_[bi, :, sl].T
        if causal:
          s = np.where(np.tril(np.ones((l, l), bool)), s, -np.inf)
        out[bi, :, sl] = scipy.special.softmax(s, axis=-1) @ v_[bi, :, sl]
    return out
  for causal in (False, True):
    dq, dk, dv = B.attention_core_backward(q, k, v, do, heads, causal)
    uq = f64(b, l, heads * d)
    for grad, which in ((dq, 0), (dk, 1), (dv, 2)):
      def loss(a, which=which):
        args = [q, k, v]
        args[which] = a
        return (core64(*args, causal) * do).sum()
      np.testing.assert_allclose((grad * uq).sum(),
                                 _fd(loss, (q, k, v)[which], uq), rtol=5e-4)
    if causal:       # the first query sees one key: a softmax of one element
      np.testing.assert_allclose(dq[:, 0], 0, atol=1e-6)
